// Small-M linear layers (decode): y[M,N] = x[M,K] . W[K,N], M <= 64, bandwidth-bound.
//
// The weight stream is read once with 128-bit loads per lane, already in MFMA operand order,
// and multiplied on the matrix cores (v_mfma_f32_16x16x32_bf16) with the activations as the
// A operand (rows = batch entries, padded to 16) and the weights as the B operand.
//
// int4: the B operand is 128+q, produced from a packed word with four and-or instructions
// (bf16 0x4300|q == 128+q exactly).  Per group of 128 rows the matrix cores give
//   T[m][n] = sum_k x[m][k]*(128+q[k][n])   and   X[m] = sum_k x[m][k]   (B = all ones)
// and the fp32 epilogue adds scale[n]*(T - (128+zero[n])*X), which equals
// sum_k x*scale*(q-zero) with the scale and zero applied in fp32.
//
// K is split over the waves of a workgroup (LDS reduction in fixed order) and optionally over
// workgroups (fp32 partials + a ticket; the last workgroup adds the partials in fixed order),
// so the result does not depend on scheduling.
#include "common.h"

namespace {

__device__ __forceinline__ bf16x8 unpack_w4_bias128(uint32_t w) {
  u32x4 r;
  r.x = (w & 0x000f000fu) | 0x43004300u;
  r.y = ((w >> 4) & 0x000f000fu) | 0x43004300u;
  r.z = ((w >> 8) & 0x000f000fu) | 0x43004300u;
  r.w = ((w >> 12) & 0x000f000fu) | 0x43004300u;
  return __builtin_bit_cast(bf16x8, r);
}

__device__ __forceinline__ bf16x8 ones_bf16x8() {
  u32x4 r = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  return __builtin_bit_cast(bf16x8, r);
}

__device__ __forceinline__ bf16x8 load_x_frag(const uint16_t* __restrict__ x, int row, int M, int K, int k) {
  if (row < M) return *reinterpret_cast<const bf16x8*>(x + (int64_t)row * K + k);
  u32x4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, z);
}

// Shared epilogue: reduce acc over the waves of the workgroup, then either write y or go
// through the cross-workgroup ticket.
template <int MT, int NT, int WAVES>
__device__ __forceinline__ void gemv_epilogue(f32x4 (&acc)[MT][NT], float* red, uint16_t* __restrict__ y,
                                              float* __restrict__ partial, unsigned* __restrict__ counters, int M, int N,
                                              int nt0, int ntiles, int ksplit) {
  constexpr int PER_WAVE = MT * NT * 256;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave * PER_WAVE + ((mt * NT + nt) * 4 + r) * 64 + lane] = acc[mt][nt][r];
  __syncthreads();
  const int s = blockIdx.y;
  const int Mp = MT * 16;
  for (int i = threadIdx.x; i < PER_WAVE; i += WAVES * 64) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) v += red[w * PER_WAVE + i];
    const int l = i & 63, r = (i >> 6) & 3, t = i >> 8;
    const int nt = t % NT, mt = t / NT;
    const int m = mt * 16 + 4 * (l >> 4) + r;
    const int n = (nt0 + nt) * 16 + (l & 15);
    if (nt0 + nt < ntiles) {
      if (ksplit == 1) {
        if (m < M) y[(int64_t)m * N + n] = f32_to_bf16_bits(v);
      } else {
        partial[((int64_t)s * Mp + m) * N + n] = v;
      }
    }
  }
  if (ksplit == 1) return;
  __shared__ int is_last;
  __threadfence();
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned t = atomicAdd(&counters[blockIdx.x], 1u);
    is_last = (t == (unsigned)(ksplit - 1));
  }
  __syncthreads();
  if (!is_last) return;
  __threadfence();
  for (int i = threadIdx.x; i < PER_WAVE; i += WAVES * 64) {
    const int l = i & 63, r = (i >> 6) & 3, t = i >> 8;
    const int nt = t % NT, mt = t / NT;
    const int m = mt * 16 + 4 * (l >> 4) + r;
    const int n = (nt0 + nt) * 16 + (l & 15);
    if (nt0 + nt < ntiles && m < M) {
      float v = 0.f;
      for (int ss = 0; ss < ksplit; ++ss)
        v += __hip_atomic_load(&partial[((int64_t)ss * Mp + m) * N + n], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      y[(int64_t)m * N + n] = f32_to_bf16_bits(v);
    }
  }
  if (threadIdx.x == 0) __hip_atomic_store(&counters[blockIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int MT, int NT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void w4_gemv_kernel(const uint16_t* __restrict__ x,
                                                             const u32x4* __restrict__ wt,
                                                             const uint16_t* __restrict__ st,
                                                             const uint8_t* __restrict__ zt, uint16_t* __restrict__ y,
                                                             float* __restrict__ partial,
                                                             unsigned* __restrict__ counters, int M, int N, int K,
                                                             int ksplit) {
  __shared__ float red[WAVES * MT * NT * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kq = lane >> 4;
  const int G = K >> 7, ntiles = N >> 4;
  const int nt0 = blockIdx.x * NT;
  const int g_begin = (int)((int64_t)G * blockIdx.y / ksplit), g_end = (int)((int64_t)G * (blockIdx.y + 1) / ksplit);
  const bf16x8 ones = ones_bf16x8();
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = zero4;

  for (int g = g_begin + wave; g < g_end; g += WAVES) {
    u32x4 w[NT];
    float sc[NT], zc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int tnt = min(nt0 + nt, ntiles - 1);  // clamp: out-of-range tiles are computed and dropped
      const int64_t tile = (int64_t)tnt * G + g;
      w[nt] = __builtin_nontemporal_load(&wt[tile * 64 + lane]);
      sc[nt] = (float)__builtin_bit_cast(_Float16, st[tile * 16 + col]);
      zc[nt] = (float)(129 + (int)((zt[tile * 8 + (col >> 1)] >> (4 * (col & 1))) & 15u));  // 128 + (stored + 1)
    }
    f32x4 t[MT][NT], xs[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      xs[mt] = zero4;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) t[mt][nt] = zero4;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      bf16x8 a[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        a[mt] = load_x_frag(x, mt * 16 + col, M, K, 128 * g + 32 * j + 8 * kq);
        xs[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[mt], ones, xs[mt], 0, 0, 0);
      }
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const bf16x8 b = unpack_w4_bias128(w[nt][j]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) t[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[mt], b, t[mt][nt], 0, 0, 0);
      }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[mt][nt][r] += sc[nt] * (t[mt][nt][r] - zc[nt] * xs[mt][r]);
  }
  gemv_epilogue<MT, NT, WAVES>(acc, red, y, partial, counters, M, N, nt0, ntiles, ksplit);
}

template <int MT, int NT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void b16_gemv_kernel(const uint16_t* __restrict__ x,
                                                              const bf16x8* __restrict__ wt, uint16_t* __restrict__ y,
                                                              float* __restrict__ partial,
                                                              unsigned* __restrict__ counters, int M, int N, int K,
                                                              int ksplit) {
  __shared__ float red[WAVES * MT * NT * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kq = lane >> 4;
  const int KS = K >> 5, ntiles = N >> 4;
  const int nt0 = blockIdx.x * NT;
  const int s_begin = (int)((int64_t)KS * blockIdx.y / ksplit), s_end = (int)((int64_t)KS * (blockIdx.y + 1) / ksplit);
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = zero4;
#pragma unroll 4
  for (int ks = s_begin + wave; ks < s_end; ks += WAVES) {
    bf16x8 b[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int tnt = min(nt0 + nt, ntiles - 1);
      b[nt] = __builtin_nontemporal_load(&wt[((int64_t)tnt * KS + ks) * 64 + lane]);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const bf16x8 a = load_x_frag(x, mt * 16 + col, M, K, 32 * ks + 8 * kq);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[nt], acc[mt][nt], 0, 0, 0);
    }
  }
  gemv_epilogue<MT, NT, WAVES>(acc, red, y, partial, counters, M, N, nt0, ntiles, ksplit);
}

constexpr int kWaves = 4;
constexpr int kCounterBytes = O355_GEMV_COUNTER_BYTES;

struct GemvPlan {
  int mt, nt, ksplit;
  unsigned blocks_x;
};

// units: number of K pieces a wave can own (groups of 128 for int4, steps of 32 for bf16)
inline GemvPlan plan_gemv(int M, int N, int units, int min_units_per_wave) {
  GemvPlan p;
  p.mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int ntiles = N >> 4;
  p.nt = (p.mt == 1 && ntiles >= 2048) ? 2 : 1;
  p.blocks_x = (unsigned)((ntiles + p.nt - 1) / p.nt);
  const int64_t target_waves = 256 * 8;
  int ks = (int)((target_waves + (int64_t)p.blocks_x * kWaves - 1) / ((int64_t)p.blocks_x * kWaves));
  const int ks_max = units / (kWaves * min_units_per_wave);
  if (ks > ks_max) ks = ks_max;
  if (ks < 1) ks = 1;
  if (ks > 8) ks = 8;
  if (p.blocks_x > (unsigned)(kCounterBytes / 4)) ks = 1;
  p.ksplit = ks;
  return p;
}

inline int64_t plan_ws_bytes(const GemvPlan& p, int N) {
  if (p.ksplit == 1) return 0;
  return (int64_t)kCounterBytes + (int64_t)p.ksplit * p.mt * 16 * N * 4;
}

#define GEMV_DISPATCH(KERNEL, MTv, NTv, ...)                                                                     \
  hipLaunchKernelGGL((KERNEL<MTv, NTv, kWaves>), dim3(p.blocks_x, p.ksplit), dim3(kWaves * 64), 0, as_stream(stream), \
                     __VA_ARGS__)

}  // namespace

extern "C" int64_t olmo355_w4_gemv_workspace_bytes(int M, int N, int K) {
  if (M <= 0 || M > 64 || N <= 0 || K <= 0 || (K & 127) || (N & 15)) return 0;
  // the dense bf16 path shares the workspace: size for whichever plan needs more
  const GemvPlan a = plan_gemv(M, N, K >> 7, 2), b = plan_gemv(M, N, K >> 5, 8);
  const int64_t wa = plan_ws_bytes(a, N), wb = plan_ws_bytes(b, N);
  return wa > wb ? wa : wb;
}

extern "C" int olmo355_w4_gemv(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                               uint16_t* y, void* ws, int M, int N, int K, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (M > 64 || (K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  const GemvPlan p = plan_gemv(M, N, K >> 7, 2);
  if (p.ksplit > 1 && !ws) return O355_EINVAL;
  unsigned* counters = (unsigned*)ws;
  float* partial = ws ? (float*)((char*)ws + kCounterBytes) : nullptr;
  const u32x4* w = (const u32x4*)wt;
  if (p.mt == 1 && p.nt == 1) GEMV_DISPATCH(w4_gemv_kernel, 1, 1, x, w, st, zt, y, partial, counters, M, N, K, p.ksplit);
  else if (p.mt == 1) GEMV_DISPATCH(w4_gemv_kernel, 1, 2, x, w, st, zt, y, partial, counters, M, N, K, p.ksplit);
  else if (p.mt == 2) GEMV_DISPATCH(w4_gemv_kernel, 2, 1, x, w, st, zt, y, partial, counters, M, N, K, p.ksplit);
  else GEMV_DISPATCH(w4_gemv_kernel, 4, 1, x, w, st, zt, y, partial, counters, M, N, K, p.ksplit);
  O355_CHECK_LAUNCH();
}

// dense bf16 small-M path; workspace rules as for olmo355_w4_gemv (same size function)
extern "C" int olmo355_b16_gemv(const uint16_t* x, const uint16_t* wt, uint16_t* y, void* ws, int M, int N, int K,
                                   void* stream) {
  if (!x || !wt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (M > 64 || (K & 31) || (N & 15)) return O355_EUNSUPPORTED;
  GemvPlan p = plan_gemv(M, N, K >> 5, 8);
  if (p.ksplit > 1 && !ws) {
    p.ksplit = 1;
  }
  unsigned* counters = (unsigned*)ws;
  float* partial = ws ? (float*)((char*)ws + kCounterBytes) : nullptr;
  const bf16x8* w = (const bf16x8*)wt;
  if (p.mt == 1 && p.nt == 1) GEMV_DISPATCH(b16_gemv_kernel, 1, 1, x, w, y, partial, counters, M, N, K, p.ksplit);
  else if (p.mt == 1) GEMV_DISPATCH(b16_gemv_kernel, 1, 2, x, w, y, partial, counters, M, N, K, p.ksplit);
  else if (p.mt == 2) GEMV_DISPATCH(b16_gemv_kernel, 2, 1, x, w, y, partial, counters, M, N, K, p.ksplit);
  else GEMV_DISPATCH(b16_gemv_kernel, 4, 1, x, w, y, partial, counters, M, N, K, p.ksplit);
  O355_CHECK_LAUNCH();
}
