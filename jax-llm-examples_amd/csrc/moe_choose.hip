// The choice of experts by scores: s = sigmoid(z), choice scores c = s + correction; with groups, the experts form
// equal groups of neighbours, a group's score is the sum of its `terms` largest c, the `keep` best groups stay; the
// top_k largest c among the experts that stay, lowest index first among equals; the weights are the chosen s.
// A thread per token walks through the experts (their number is small beside a token's other work).  And the
// experts' activation relu(x)^2, element by element.
#include "common.h"

using namespace jle;

namespace {

constexpr int kMaxGroups = 64, kMaxTerms = 4, kMaxTop = 16, kCached = 64;

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

__global__ __launch_bounds__(64) void moe_choose_kernel(const float* __restrict__ logits,
                                                        const float* __restrict__ correction, int* __restrict__ ids,
                                                        float* __restrict__ weights, int N, int E, int top_k,
                                                        int groups, int keep, int terms) {
  // (a thread's lists lie in shared memory: indexed by values that are known only when the kernel runs, they would
  // otherwise be kept in scratch memory)
  __shared__ float score_all[kMaxGroups][64];
  __shared__ int chosen_all[kMaxTop][64];
  const int n = blockIdx.x * 64 + threadIdx.x;
  if (n >= N) return;
  const int me = threadIdx.x;
  const float* z = logits + (size_t)n * E;
  // the choice scores of up to kCached experts are formed once and kept in shared memory (a thread walks through them
  // top_k + 1 times); with more experts they are formed anew each time
  __shared__ float cached[kCached][64];
  const bool in_lds = E <= kCached;
  if (in_lds)
    for (int e = 0; e < E; ++e) cached[e][me] = sigmoidf_(z[e]) + (correction != nullptr ? correction[e] : 0.f);
  auto choice = [&](int e) {
    return in_lds ? cached[e][me] : sigmoidf_(z[e]) + (correction != nullptr ? correction[e] : 0.f);
  };
  unsigned long long kept = ~0ull;  // bit gi: group gi's experts can be chosen
  const int per = groups > 0 ? E / groups : E;
  if (groups > 0) {
    for (int gi = 0; gi < groups; ++gi) {
      float best[kMaxTerms];
#pragma unroll
      for (int i = 0; i < kMaxTerms; ++i) best[i] = -INFINITY;
      for (int e = gi * per; e < (gi + 1) * per; ++e) {
        float c = choice(e);
#pragma unroll
        for (int i = 0; i < kMaxTerms; ++i) {  // (kept in descending order)
          if (i < terms && c > best[i]) {
            const float t = best[i];
            best[i] = c;
            c = t;
          }
        }
      }
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < kMaxTerms; ++i)
        if (i < terms && i < per) sum += best[i];
      score_all[gi][me] = sum;
    }
    kept = 0ull;
    for (int r = 0; r < keep; ++r) {
      int at = -1;
      float top = 0.f;
      for (int gi = 0; gi < groups; ++gi) {
        if ((kept >> gi) & 1ull) continue;
        const float sc = score_all[gi][me];
        if (at < 0 || sc > top) {
          at = gi;
          top = sc;
        }
      }
      kept |= 1ull << at;
    }
  }
  for (int r = 0; r < top_k; ++r) {
    int at = -1;
    float top = 0.f;
    for (int e = 0; e < E; ++e) {
      if (groups > 0 && !((kept >> (e / per)) & 1ull)) continue;
      bool taken = false;
      for (int i = 0; i < r; ++i) taken |= chosen_all[i][me] == e;
      if (taken) continue;
      const float c = choice(e);
      if (at < 0 || c > top) {
        at = e;
        top = c;
      }
    }
    chosen_all[r][me] = at;
    ids[(size_t)n * top_k + r] = at;
    weights[(size_t)n * top_k + r] = sigmoidf_(z[at]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void relu2_kernel(const T* __restrict__ x, T* __restrict__ y, long long count) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  const float v = fmaxf(Num<T>::load(x + i), 0.f);
  Num<T>::store(y + i, v * v);
}

}  // namespace

// groups == 0: no groups.  logits float32 [N, E]; correction float32 [E] or null.
JLE_API int jle_moe_choose(const float* logits, const float* correction, int* ids, float* weights, int N, int E,
                           int top_k, int groups, int keep, int terms, hipStream_t s) {
  if (N <= 0) return 0;
  if (logits == nullptr || ids == nullptr || weights == nullptr || E <= 0 || top_k < 1 || top_k > kMaxTop || top_k > E)
    return JLE_BAD_ARG;
  if (groups < 0 || groups > kMaxGroups ||
      (groups > 0 && (E % groups || keep < 1 || keep > groups || terms < 1 || terms > kMaxTerms ||
                      keep * (E / groups) < top_k)))
    return JLE_BAD_ARG;
  hipLaunchKernelGGL(moe_choose_kernel, dim3((N + 63) / 64), dim3(64), 0, s, logits, correction, ids, weights, N, E,
                     top_k, groups, keep, terms);
  JLE_LAUNCH_CHECK();
  return 0;
}

JLE_API int jle_relu2(const void* x, void* y, int is_bf16, long long count, hipStream_t s) {
  if (count <= 0) return 0;
  if (x == nullptr || y == nullptr || (count + 255) / 256 > 2147483647LL) return JLE_BAD_ARG;
  if (is_bf16)
    hipLaunchKernelGGL(relu2_kernel<bf16_t>, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, (const bf16_t*)x,
                       (bf16_t*)y, count);
  else
    hipLaunchKernelGGL(relu2_kernel<float>, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, (const float*)x,
                       (float*)y, count);
  JLE_LAUNCH_CHECK();
  return 0;
}
