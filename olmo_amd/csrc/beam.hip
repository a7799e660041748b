// Beam search on the device (olmo/beam_search.py:813-1045 with the deterministic sampler, :102-113): the two
// selections of a step, each one workgroup per row.
//   log_softmax: the step function's normalisation (olmo/model.py:1705), activation-dtype logits in, fp32
//                log-probabilities out (the reference keeps them in the activation dtype; fp32 loses nothing).
//   topk:        the k largest of a row in descending order, equal values in ascending index order
//                (torch.topk leaves the order of ties open; with k = 1 this is torch.argmax's rule).
//                Used for the per-node candidates (rows = batch * beam, n = vocabulary) and for the
//                beam-level cut (rows = batch, n = beam * per_node_beam_size).
// Selection is k rounds of a lexicographic arg-max over the row, which stays in L2 between rounds: beam widths
// are single digits, and the rounds are exact and independent of scheduling.
#include <math.h>

#include "common.h"

namespace {

constexpr int kThreads = 1024, kWaves = kThreads / 64;

__device__ __forceinline__ float block_max_f(float v, float* lds) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = lds[0];
  for (int i = 1; i < kWaves; ++i) t = fmaxf(t, lds[i]);
  return t;
}

__device__ __forceinline__ float block_sum_f(float v, float* lds) {  // fixed order: result independent of timing
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = lds[0];
  for (int i = 1; i < kWaves; ++i) t += lds[i];
  return t;
}

template <int DT>
__global__ __launch_bounds__(kThreads) void log_softmax_kernel(const void* __restrict__ x, float* __restrict__ out,
                                                               int n) {
  __shared__ float red[kWaves];
  const int64_t base = (int64_t)blockIdx.x * n;
  float m = -INFINITY;
  for (int i = threadIdx.x; i < n; i += kThreads) m = fmaxf(m, Act<DT>::ld(x, base + i));
  m = block_max_f(m, red);
  float s = 0.f;
  for (int i = threadIdx.x; i < n; i += kThreads) s += expf(Act<DT>::ld(x, base + i) - m);
  s = block_sum_f(s, red);
  const float lse = logf(s);
  for (int i = threadIdx.x; i < n; i += kThreads) out[base + i] = (Act<DT>::ld(x, base + i) - m) - lse;
}

// (a, ia) before (b, ib) in the output order: larger value first, then smaller index
__device__ __forceinline__ bool before(float a, int ia, float b, int ib) { return a > b || (a == b && ia < ib); }

__global__ __launch_bounds__(kThreads) void topk_kernel(const float* __restrict__ x, int n, int k,
                                                        float* __restrict__ out_v, int64_t* __restrict__ out_i) {
  __shared__ float sv[kWaves];
  __shared__ int si[kWaves];
  __shared__ float pick_v;
  __shared__ int pick_i;
  const int64_t base = (int64_t)blockIdx.x * n;
  float prev_v = INFINITY;
  int prev_i = -1;
  for (int r = 0; r < k; ++r) {
    float best = -INFINITY;
    int bi = 0x7fffffff;  // nothing yet
    for (int i = threadIdx.x; i < n; i += kThreads) {
      const float v = x[base + i];
      // still to be emitted: strictly after the previous pick in the output order
      if (before(prev_v, prev_i, v, i) && before(v, i, best, bi)) best = v, bi = i;
    }
    wave_first_pair(best, bi, [](float ov, int oi, float v, int i) { return before(ov, oi, v, i); });
    if ((threadIdx.x & 63) == 0) sv[threadIdx.x >> 6] = best, si[threadIdx.x >> 6] = bi;
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int w = 1; w < kWaves; ++w)
        if (before(sv[w], si[w], best, bi)) best = sv[w], bi = si[w];
      pick_v = best, pick_i = bi;
      out_v[(int64_t)blockIdx.x * k + r] = best;
      out_i[(int64_t)blockIdx.x * k + r] = bi == 0x7fffffff ? 0 : bi;  // only when the row holds NaNs
    }
    __syncthreads();
    prev_v = pick_v, prev_i = pick_i;
  }
}

__host__ __device__ __forceinline__ uint64_t mix64(uint64_t x) {  // splitmix64 finaliser
  x += 0x9e3779b97f4a7c15ull;
  x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
  x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
  return x ^ (x >> 31);
}

// out = x * inv_temp + G with G ~ Gumbel(0, 1) drawn from (seed, counter, row, column); entries at or below half
// the float minimum (what the search uses for "impossible") become -inf.  The k largest of a perturbed row are k
// draws without replacement from softmax(x * inv_temp) (the Gumbel-top-k property), which is how
// torch.multinomial(probabilities, k) of the reference's samplers (olmo/beam_search.py:135-146, 171-203, 238-289) is
// realised here; k launches with different counters and k = 1 give draws with replacement.
__global__ __launch_bounds__(256) void gumbel_perturb_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                             int64_t total, int n, float inv_temp, uint64_t seed,
                                                             uint64_t counter) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const float v = x[i];
  if (!(v > -1.7e38f)) {
    out[i] = -INFINITY;
    return;
  }
  const uint64_t r = mix64(mix64(seed ^ (counter * 0xd1342543de82ef95ull)) + (uint64_t)i);
  const float u = ((float)(uint32_t)(r >> 40) + 0.5f) * (1.f / 16777216.f);  // (0, 1), 24 bits
  out[i] = v * inv_temp - logf(-logf(u));
}

__device__ __forceinline__ float gumbel_at(float phi, uint64_t key, int64_t i) {
  if (!(phi > -1.7e38f)) return -INFINITY;
  const uint64_t r = mix64(key + (uint64_t)i);
  const float u = ((float)(uint32_t)(r >> 40) + 0.5f) * (1.f / 16777216.f);
  return phi - logf(-logf(u));
}

// Gumbel(phi) per element conditioned on the row maximum being T[row] (GumbelSampler.gumbel_with_max,
// olmo/beam_search.py:403-421): G = phi + noise, Z = max G, v = T - G + log1p(-exp(G - Z)),
// out = T - max(v, 0) - log1p(exp(-|v|)).  One workgroup per row; the noise is regenerated for the second pass
// instead of being stored.
__global__ __launch_bounds__(kThreads) void gumbel_with_max_kernel(const float* __restrict__ phi,
                                                                   const float* __restrict__ t_row,
                                                                   float* __restrict__ out, int n, uint64_t key) {
  __shared__ float red[kWaves];
  const int64_t base = (int64_t)blockIdx.x * n;
  float z = -INFINITY;
  for (int i = threadIdx.x; i < n; i += kThreads) z = fmaxf(z, gumbel_at(phi[base + i], key, base + i));
  z = block_max_f(z, red);
  const float t = t_row[blockIdx.x];
  for (int i = threadIdx.x; i < n; i += kThreads) {
    const float g = gumbel_at(phi[base + i], key, base + i);
    const float v = t - g + log1pf(-expf(g - z));
    out[base + i] = t - fmaxf(v, 0.f) - log1pf(expf(-fabsf(v)));
  }
}

}  // namespace

extern "C" int olmo355_gumbel_with_max(const float* phi, const float* row_max, float* out, int rows, int n, uint64_t seed,
                                       uint64_t counter, void* stream) {
  if (!phi || !row_max || !out || rows <= 0 || n <= 0) return O355_EINVAL;
  hipLaunchKernelGGL(gumbel_with_max_kernel, dim3(rows), dim3(kThreads), 0, as_stream(stream), phi, row_max, out, n,
                     mix64(seed ^ (counter * 0xd1342543de82ef95ull)));
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_gumbel_perturb(const float* x, float* out, int rows, int n, float inv_temp, uint64_t seed,
                                      uint64_t counter, void* stream) {
  if (!x || !out || rows <= 0 || n <= 0 || !(inv_temp > 0.f)) return O355_EINVAL;
  const int64_t total = (int64_t)rows * n;
  hipLaunchKernelGGL(gumbel_perturb_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, as_stream(stream), x, out,
                     total, n, inv_temp, seed, counter);
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_log_softmax(const void* logits, float* out, int rows, int n, int dtype, void* stream) {
  if (!logits || !out || rows <= 0 || n <= 0) return O355_EINVAL;
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case O355_F32: hipLaunchKernelGGL(log_softmax_kernel<O355_F32>, dim3(rows), dim3(kThreads), 0, s, logits, out, n); break;
    case O355_BF16: hipLaunchKernelGGL(log_softmax_kernel<O355_BF16>, dim3(rows), dim3(kThreads), 0, s, logits, out, n); break;
    case O355_F16: hipLaunchKernelGGL(log_softmax_kernel<O355_F16>, dim3(rows), dim3(kThreads), 0, s, logits, out, n); break;
    default: return O355_EUNSUPPORTED;
  }
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_topk(const float* x, int rows, int n, int k, float* out_vals, int64_t* out_idx, void* stream) {
  if (!x || !out_vals || !out_idx || rows <= 0 || n <= 0 || k <= 0 || k > n) return O355_EINVAL;
  if (k > 1024) return O355_EUNSUPPORTED;  // k passes over the row: meant for beam widths
  hipLaunchKernelGGL(topk_kernel, dim3(rows), dim3(kThreads), 0, as_stream(stream), x, n, k, out_vals, out_idx);
  O355_CHECK_LAUNCH();
}
