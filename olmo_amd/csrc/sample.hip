// One sampling step on the device: temperature, top-k and top-p filters and the draw, one workgroup per
// row of logits, so a sampled decode step stays inside the captured graph like the greedy one.
//
// What is sampled (olmo/beam_search.py with beam size 1): with z = logits / temperature and
// e_i = exp(z_i - max z),
//   MultinomialSampler (:117-146)  draws i with probability e_i / sum(e);
//   TopKSampler (:149-196)         keeps the k largest e_i;
//   TopPSampler (:199-277)         sorts descending and keeps tokens up to and including the one at which
//                                  the cumulative probability first reaches p;
// and the returned score is log_softmax(logits)[i] at temperature 1 (the gather from the unscaled
// log-probabilities, :146,196,277).  Here both filters are thresholds on e: the largest t with
// count(e >= t) >= k, and the largest t with mass(e >= t) >= p * mass(kept).  Tokens tied with the
// threshold are all kept, where torch.topk / torch.sort keep an arbitrary subset of them.  The
// threshold is found by a radix select, 4 bits per pass (histograms of integer counts and 2^-32 fixed-point
// masses: every sum is exact, so the result does not depend on scheduling); after the first pass or two
// the tokens still in range fit LDS and the remaining passes no longer read the row.
// The draw walks the kept tokens in a fixed order (thread by thread, each in its own visiting order) with one 64-bit uniform number from
// splitmix64(seed, counter, row): the distribution is the reference's, its random stream is not.
#include "common.h"
#include <type_traits>

namespace {

constexpr int kThreads = 1024, kWaves = kThreads / 64;

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
  x += 0x9e3779b97f4a7c15ull;
  x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
  x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
  return x ^ (x >> 31);
}

// sum over the wave of a 64-bit count per lane, in every lane: the butterfly of wave_sum on both halves (register
// moves, no trips through the LDS crossbar; integer sums do not depend on the order)
__device__ __forceinline__ uint64_t wave_sum_u64(uint64_t v) {
  auto join = [](uint32_t lo, uint32_t hi) { return ((uint64_t)hi << 32) | lo; };
  auto dpp_step = [&](auto ctrl) {
    constexpr int C = decltype(ctrl)::value;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)v, C, 0xF, 0xF, true);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(v >> 32), C, 0xF, 0xF, true);
    v += join(lo, hi);
  };
  dpp_step(std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
  dpp_step(std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]
  dpp_step(std::integral_constant<int, 0x141>{});  // row_half_mirror (the quads agree by now)
  dpp_step(std::integral_constant<int, 0x140>{});  // row_mirror
  {
    const auto lo = __builtin_amdgcn_permlane16_swap((uint32_t)v, (uint32_t)v, false, false);
    const auto hi = __builtin_amdgcn_permlane16_swap((uint32_t)(v >> 32), (uint32_t)(v >> 32), false, false);
    v = join(lo[0], hi[0]) + join(lo[1], hi[1]);
  }
  {
    const auto lo = __builtin_amdgcn_permlane32_swap((uint32_t)v, (uint32_t)v, false, false);
    const auto hi = __builtin_amdgcn_permlane32_swap((uint32_t)(v >> 32), (uint32_t)(v >> 32), false, false);
    v = join(lo[0], hi[0]) + join(lo[1], hi[1]);
  }
  return v;
}

// sum of NV 64-bit values per thread over the workgroup; every thread gets the totals
template <int NV>
__device__ __forceinline__ void block_sum_u64(uint64_t (&v)[NV], uint64_t* lds /* [kWaves][NV] */) {
#pragma unroll
  for (int j = 0; j < NV; ++j) v[j] = wave_sum_u64(v[j]);
  const int w = threadIdx.x >> 6;
  __syncthreads();  // the previous use of lds is over
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int j = 0; j < NV; ++j) lds[w * NV + j] = v[j];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    uint64_t t = 0;
    for (int i = 0; i < kWaves; ++i) t += lds[i * NV + j];
    v[j] = t;
  }
}

__device__ __forceinline__ float block_max(float v, float* lds /* [kWaves] */) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = lds[0];
  for (int i = 1; i < kWaves; ++i) t = fmaxf(t, lds[i]);
  return t;
}

// Once a search has narrowed the tokens that can still hold the threshold to kCap or fewer, they are
// copied into LDS and the remaining passes run there instead of over the row.
constexpr int kCap = 8192;

// exclusive scan of one 64-bit value per thread; returns the total
__device__ __forceinline__ uint64_t block_scan_u64(uint64_t mine, uint64_t* scan /* [kThreads] */, uint64_t& excl) {
  const int tid = threadIdx.x;
  __syncthreads();
  scan[tid] = mine;
  __syncthreads();
  for (int o = 1; o < kThreads; o <<= 1) {
    const uint64_t v = tid >= o ? scan[tid - o] : 0ull;
    __syncthreads();
    scan[tid] += v;
    __syncthreads();
  }
  excl = scan[tid] - mine;
  return scan[kThreads - 1];
}

template <int DT>
__global__ __launch_bounds__(kThreads) void sample_kernel(const void* __restrict__ logits, int n, float inv_temp,
                                                          int top_k, float top_p, uint64_t seed,
                                                          const int32_t* __restrict__ counter_dev, int counter,
                                                          int64_t* __restrict__ out, float* __restrict__ logprob) {
  __shared__ uint64_t red[kWaves * 2];
  __shared__ float redf[kWaves];
  __shared__ uint64_t scan[kThreads];
  __shared__ uint32_t h_cnt[kWaves][16];
  __shared__ uint64_t h_mass[kWaves][16];
  __shared__ uint32_t t_cnt[16];
  __shared__ uint64_t t_mass[16];
  __shared__ uint32_t cand_key[kCap];
  __shared__ uint32_t cand_n;
  const int tid = threadIdx.x, row = blockIdx.x, wave = tid >> 6;
  const int64_t base = (int64_t)row * n;

  // Every pass over the row visits the tokens in the same per-thread order: f(i, logit_i) -> false stops the
  // thread's walk.  bf16 rows whose length is a multiple of 8 are read 16 bytes per lane.
  const bool vec = DT == O355_BF16 && (n & 7) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0;
  auto for_each = [&](auto f) {
    if (vec) {
      const u32x4* src = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(logits) + base);
      for (int v = tid; v < (n >> 3); v += kThreads) {
        const u32x4 x = src[v];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint32_t w = x[e >> 1];
          if (!f(v * 8 + e, (e & 1) ? bf16hi_to_f32(w) : bf16lo_to_f32(w))) return;
        }
      }
    } else {
      for (int i = tid; i < n; i += kThreads)
        if (!f(i, Act<DT>::ld(logits, base + i))) return;
    }
  };

  // ---- maxima (no exponentials yet)
  float mz = -INFINITY, m1 = -INFINITY;
  for_each([&](int, float l) {
    m1 = fmaxf(m1, l), mz = fmaxf(mz, l * inv_temp);
    return true;
  });
  mz = block_max(mz, redf);
  m1 = block_max(m1, redf);

  // e_i in (0, 1] as a float key (monotone as an unsigned integer) and as 2^-32 fixed point; one fma and one
  // hardware exp2 per evaluation: the same bits every time it is evaluated, which is all the passes need
  const float c2 = inv_temp * 1.4426950408889634f, mz2 = mz * 1.4426950408889634f;
  auto key_of = [&](float l) { return __float_as_uint(__builtin_amdgcn_exp2f(__builtin_fmaf(l, c2, -mz2))); };
  auto mass_of = [](uint32_t key) { return (uint64_t)(__uint_as_float(key) * 4294967296.f); };

  // ---- one pass: normaliser of the unscaled distribution (the returned log-probability), this thread's mass
  float s1 = 0.f;
  uint64_t my_mass = 0;
  for_each([&](int, float l) {
    s1 += expf(l - m1);
    my_mass += mass_of(key_of(l));
    return true;
  });
  s1 = wave_sum(s1);
  __syncthreads();
  if ((tid & 63) == 0) redf[wave] = s1;
  __syncthreads();
  s1 = 0.f;
  for (int i = 0; i < kWaves; ++i) s1 += redf[i];  // fixed order
  const float lse1 = m1 + logf(s1);

  // ---- radix select: the largest threshold t with F(key >= t) >= target among the tokens with key >=
  // floor_key, F = their number (top-k) or their mass (top-p).  Four bits per pass, most significant first:
  // a histogram of the tokens still in range (per-wave LDS counters, integer adds: exact in any order), then
  // the bucket at which the running total from the top reaches the target becomes the new range.
  auto select = [&](bool by_mass, uint64_t target, uint32_t floor_key) {
    uint32_t prefix = 0;
    uint64_t above = 0;
    bool in_lds = false;
    int src_n = n;
    for (int shift = 28; shift >= 0; shift -= 4) {
      const uint32_t hi_mask = shift == 28 ? 0u : ~0u << (shift + 4);
      __syncthreads();
      if (tid < kWaves * 16) (&h_cnt[0][0])[tid] = 0u, (&h_mass[0][0])[tid] = 0ull;
      __syncthreads();
      // a thread adds up runs of tokens that fall into the same bucket before touching the shared counters:
      // in the leading passes nearly every token shares its top bits with the rest
      int run_b = 0;
      uint32_t run_c = 0;
      uint64_t run_m = 0;
      auto flush = [&]() {
        if (run_c) {
          atomicAdd(&h_cnt[wave][run_b], run_c);
          if (by_mass) atomicAdd(reinterpret_cast<unsigned long long*>(&h_mass[wave][run_b]), (unsigned long long)run_m);
        }
      };
      auto visit = [&](uint32_t key) {
        if (key < floor_key || (key & hi_mask) != prefix) return;
        const int b = (key >> shift) & 15;
        if (b != run_b) flush(), run_b = b, run_c = 0, run_m = 0;
        run_c += 1;
        if (by_mass) run_m += mass_of(key);
      };
      if (in_lds) {
        for (int i = tid; i < src_n; i += kThreads) visit(cand_key[i]);
      } else {
        for_each([&](int, float l) {
          visit(key_of(l));
          return true;
        });
      }
      flush();
      __syncthreads();
      if (tid < 16) {
        uint32_t c = 0;
        uint64_t m = 0;
        for (int w = 0; w < kWaves; ++w) c += h_cnt[w][tid], m += h_mass[w][tid];
        t_cnt[tid] = c, t_mass[tid] = m;
      }
      __syncthreads();
      int pick = 0;
      uint64_t cum = above;
      for (int b = 15; b >= 0; --b) {
        const uint64_t f = by_mass ? t_mass[b] : (uint64_t)t_cnt[b];
        if (cum + f >= target) { pick = b; break; }
        cum += f;
      }
      above = cum;
      prefix |= (uint32_t)pick << shift;
      const int active = (int)t_cnt[pick];
      if (!in_lds && shift > 0 && active <= kCap) {  // copy what is still in range into LDS (workgroup-uniform branch)
        const uint32_t nmask = ~0u << shift;
        if (tid == 0) cand_n = 0;
        __syncthreads();
        // few tokens are left in range: one LDS counter hands out the slots (the order does not matter, only sums
        // are taken over the copies)
        for_each([&](int, float l) {
          const uint32_t key = key_of(l);
          if (key >= floor_key && (key & nmask) == prefix) cand_key[atomicAdd(&cand_n, 1u)] = key;
          return true;
        });
        __syncthreads();
        in_lds = true;
        src_n = active;
      }
    }
    return prefix;
  };

  const bool want_k = top_k > 0 && top_k < n, want_p = top_p < 1.f;
  uint32_t thr = 0;  // keep everything
  if (want_k) thr = select(false, (uint64_t)top_k, 0u);
  if (want_p) {
    uint64_t kept[2] = {0, 0};
    for_each([&](int, float l) {
      const uint32_t key = key_of(l);
      kept[0] += key >= thr ? mass_of(key) : 0ull;
      return true;
    });
    block_sum_u64<2>(kept, red);
    // the reference compares cumulative probabilities with p: mass >= p * total, at least the largest token
    uint64_t target = (uint64_t)((double)fmaxf(top_p, 0.f) * (double)kept[0]);
    target = target < 1 ? 1 : target;
    const uint32_t t2 = select(true, target, thr);
    thr = t2 > thr ? t2 : thr;
  }

  // ---- the draw: kept tokens thread by thread, each in its visiting order, with one uniform number
  uint64_t mine = 0;
  if (!want_k && !want_p) {
    mine = my_mass;
  } else {
    for_each([&](int, float l) {
      const uint32_t key = key_of(l);
      mine += key >= thr ? mass_of(key) : 0ull;
      return true;
    });
  }
  uint64_t excl;
  const uint64_t total = block_scan_u64(mine, scan, excl);
  const int c = counter_dev ? *counter_dev : counter;
  const uint64_t rnd = splitmix64(splitmix64(seed ^ ((uint64_t)(uint32_t)c << 32)) + (uint64_t)row);
  const uint64_t target = __umul64hi(total, rnd);  // floor(total * u), u in [0, 1): < total
  if (total == 0) {  // cannot happen (the maximum has mass 2^32), kept for safety: the first token
    if (tid == 0) out[row] = 0, logprob[row] = Act<DT>::ld(logits, base) - lse1;
    return;
  }
  if (target >= excl && target < excl + mine) {  // exactly one thread
    uint64_t acc = excl;
    int pick = -1;
    for_each([&](int i, float l) {
      const uint32_t key = key_of(l);
      if (key < thr) return true;
      acc += mass_of(key);
      if (acc > target) pick = i;
      return pick < 0;
    });
    out[row] = pick;
    logprob[row] = Act<DT>::ld(logits, base + pick) - lse1;
  }
}

}  // namespace

extern "C" int olmo355_sample(const void* logits, int rows, int n, float temperature, int top_k, float top_p,
                              uint64_t seed, const int32_t* counter_dev, int counter, int64_t* out, float* logprob,
                              int dtype, void* stream) {
  if (!logits || !out || !logprob || rows <= 0 || n <= 0) return O355_EINVAL;
  if (!(temperature > 0.f) || top_k < 0 || !(top_p >= 0.f) || top_p > 1.f) return O355_EINVAL;
  const float inv_temp = 1.f / temperature;
  if (dtype == O355_F32)
    hipLaunchKernelGGL(sample_kernel<O355_F32>, dim3(rows), dim3(kThreads), 0, as_stream(stream), logits, n, inv_temp, top_k,
                       top_p, seed, counter_dev, counter, out, logprob);
  else if (dtype == O355_BF16)
    hipLaunchKernelGGL(sample_kernel<O355_BF16>, dim3(rows), dim3(kThreads), 0, as_stream(stream), logits, n, inv_temp,
                       top_k, top_p, seed, counter_dev, counter, out, logprob);
  else if (dtype == O355_F16)
    hipLaunchKernelGGL(sample_kernel<O355_F16>, dim3(rows), dim3(kThreads), 0, as_stream(stream), logits, n, inv_temp,
                       top_k, top_p, seed, counter_dev, counter, out, logprob);
  else
    return O355_EUNSUPPORTED;
  O355_CHECK_LAUNCH();
}
