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
// K is split over the waves of a workgroup only (contiguous slice per wave, LDS reduction in
// fixed order): no atomics, no cross-workgroup pass, so the result does not depend on scheduling.
// Each wave keeps U one-KiB weight pieces in flight and refills a slot as soon as it is consumed.
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

// Reduce acc over the waves of the workgroup in fixed order and write y (bf16).
template <int MT, int NT, int WAVES>
__device__ __forceinline__ void gemv_epilogue(f32x4 (&acc)[MT][NT], float* red, uint16_t* __restrict__ y, int M, int N,
                                              int nt0, int ntiles) {
  constexpr int PER_WAVE = MT * NT * 256;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave * PER_WAVE + ((mt * NT + nt) * 4 + r) * 64 + lane] = acc[mt][nt][r];
  __syncthreads();
  for (int i = threadIdx.x; i < PER_WAVE; i += WAVES * 64) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) v += red[w * PER_WAVE + i];
    const int l = i & 63, r = (i >> 6) & 3, t = i >> 8;
    const int nt = t % NT, mt = t / NT;
    const int m = mt * 16 + 4 * (l >> 4) + r;
    const int n = (nt0 + nt) * 16 + (l & 15);
    if (nt0 + nt < ntiles && m < M) y[(int64_t)m * N + n] = f32_to_bf16_bits(v);
  }
}

// Activation fragments.  XLDS: the workgroup first copies its M rows of x into LDS (plus one
// zero row that the padding lanes read), and every A operand is one ds_read_b128 issued right
// before its MFMA; otherwise the fragments come from global memory with the weight loads.
template <bool XLDS>
struct XSource {
  const uint16_t* x;
  const uint16_t* lds;  // [M+1][K] when XLDS
  int M, K, row_off;    // row_off: element offset of this lane's row in LDS
  __device__ __forceinline__ bf16x8 frag(int mt, int col, int k) const {
    if constexpr (XLDS) {
      return *reinterpret_cast<const bf16x8*>(lds + row_off + k);
    } else {
      return load_x_frag(x, mt * 16 + col, M, K, k);
    }
  }
};

// Copy of the M activation rows into LDS in two halves around the weight prologue: the global
// loads go out first, the LDS writes (and the barrier) come after the weight loads were issued.
constexpr int kXStageRegs = 4;
template <int WAVES, bool XLDS>
__device__ __forceinline__ void stage_x_begin(u32x4 (&xr)[kXStageRegs], const uint16_t* __restrict__ x, int M, int K) {
  if constexpr (XLDS) {
    const int total = (M * K) >> 3;  // 16-byte pieces
#pragma unroll
    for (int i = 0; i < kXStageRegs; ++i) {
      const int idx = threadIdx.x + i * WAVES * 64;
      if (idx < total) xr[i] = reinterpret_cast<const u32x4*>(x)[idx];
    }
  }
}
template <int WAVES, bool XLDS>
__device__ __forceinline__ void stage_x_finish(u32x4 (&xr)[kXStageRegs], const uint16_t* __restrict__ x, uint16_t* xl, int M,
                                               int K) {
  if constexpr (XLDS) {
    const int total = (M * K) >> 3;
#pragma unroll
    for (int i = 0; i < kXStageRegs; ++i) {
      const int idx = threadIdx.x + i * WAVES * 64;
      if (idx < total) reinterpret_cast<u32x4*>(xl)[idx] = xr[i];
    }
    for (int idx = threadIdx.x + kXStageRegs * WAVES * 64; idx < total; idx += WAVES * 64)
      reinterpret_cast<u32x4*>(xl)[idx] = reinterpret_cast<const u32x4*>(x)[idx];
    for (int i = threadIdx.x; i < (K >> 3); i += WAVES * 64)
      reinterpret_cast<u32x4*>(xl + (int64_t)M * K)[i] = u32x4{0u, 0u, 0u, 0u};
    lds_barrier();
  }
}

template <int MT, int NT, int WAVES, int U, bool XLDS>
__global__ __launch_bounds__(WAVES * 64) void w4_gemv_kernel(const uint16_t* __restrict__ x,
                                                             const u32x4* __restrict__ wt,
                                                             const uint16_t* __restrict__ st,
                                                             const uint8_t* __restrict__ zt, uint16_t* __restrict__ y,
                                                             int M, int N, int K) {
  extern __shared__ __align__(16) unsigned char smem[];
  float* red = reinterpret_cast<float*>(smem);                                         // [WAVES][MT*NT*256]
  uint16_t* xl = reinterpret_cast<uint16_t*>(smem + WAVES * MT * NT * 256 * sizeof(float));  // [M+1][K]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kq = lane >> 4;
  const int G = K >> 7, ntiles = N >> 4;
  const int nt0 = blockIdx.x * NT;
  // contiguous slice of groups per wave
  const int g_begin = (int)((int64_t)G * wave / WAVES), g_end = (int)((int64_t)G * (wave + 1) / WAVES);
  const bf16x8 ones = ones_bf16x8();
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

  static_assert(!XLDS || MT == 1, "x in LDS is for M <= 16");
  XSource<XLDS> xs_src{x, xl, M, K, (col < M ? col : M) * K};

  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = zero4;

  u32x4 w[U][NT];
  uint16_t s16[U][NT];
  uint8_t z8[U][NT];
  bf16x8 a[XLDS ? 1 : U][4][MT];

  auto issue = [&](int u, int g) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int tnt = min(nt0 + nt, ntiles - 1);  // out-of-range tiles are computed and dropped
      const int64_t tile = (int64_t)tnt * G + g;
      w[u][nt] = __builtin_nontemporal_load(&wt[tile * 64 + lane]);
      s16[u][nt] = st[tile * 16 + col];
      z8[u][nt] = zt[tile * 8 + (col >> 1)];
    }
    if constexpr (!XLDS) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) a[u][j][mt] = xs_src.frag(mt, col, 128 * g + 32 * j + 8 * kq);
    }
  };

  // x first (it comes from L2 and is needed first), then U weight pieces in flight
  u32x4 xr[kXStageRegs];
  stage_x_begin<WAVES, XLDS>(xr, x, M, K);
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (g_begin + u < g_end) issue(u, g_begin + u);

  stage_x_finish<WAVES, XLDS>(xr, x, xl, M, K);

  for (int base = g_begin; base < g_end; base += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int g = base + u;
      if (g < g_end) {
        f32x4 t[MT][NT], xsum[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          xsum[mt] = zero4;
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) t[mt][nt] = zero4;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          bf16x8 af[MT];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            if constexpr (XLDS) af[mt] = xs_src.frag(mt, col, 128 * g + 32 * j + 8 * kq);
            else af[mt] = a[u][j][mt];
            xsum[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[mt], ones, xsum[mt], 0, 0, 0);
          }
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            const bf16x8 b = unpack_w4_bias128(w[u][nt][j]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              t[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[mt], b, t[mt][nt], 0, 0, 0);
          }
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const float sc = (float)__builtin_bit_cast(_Float16, s16[u][nt]);
          const float zc = (float)(129 + (int)((z8[u][nt] >> (4 * (col & 1))) & 15u));  // 128 + (stored + 1)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[mt][nt][r] += sc * (t[mt][nt][r] - zc * xsum[mt][r]);
        }
        if (g + U < g_end) issue(u, g + U);  // refill the slot just consumed
      }
    }
  }
  gemv_epilogue<MT, NT, WAVES>(acc, red, y, M, N, nt0, ntiles);
}

template <int MT, int NT, int WAVES, int U, bool XLDS>
__global__ __launch_bounds__(WAVES * 64) void b16_gemv_kernel(const uint16_t* __restrict__ x,
                                                              const bf16x8* __restrict__ wt, uint16_t* __restrict__ y,
                                                              int M, int N, int K) {
  extern __shared__ __align__(16) unsigned char smem[];
  float* red = reinterpret_cast<float*>(smem);
  uint16_t* xl = reinterpret_cast<uint16_t*>(smem + WAVES * MT * NT * 256 * sizeof(float));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kq = lane >> 4;
  const int KS = K >> 5, ntiles = N >> 4;
  const int nt0 = blockIdx.x * NT;
  const int s_begin = (int)((int64_t)KS * wave / WAVES), s_end = (int)((int64_t)KS * (wave + 1) / WAVES);
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  static_assert(!XLDS || MT == 1, "x in LDS is for M <= 16");
  XSource<XLDS> xs_src{x, xl, M, K, (col < M ? col : M) * K};
  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = zero4;
  bf16x8 b[U][NT], a[XLDS ? 1 : U][MT];
  auto issue = [&](int u, int ks) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int tnt = min(nt0 + nt, ntiles - 1);
      b[u][nt] = __builtin_nontemporal_load(&wt[((int64_t)tnt * KS + ks) * 64 + lane]);
    }
    if constexpr (!XLDS) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) a[u][mt] = xs_src.frag(mt, col, 32 * ks + 8 * kq);
    }
  };
  u32x4 xr[kXStageRegs];
  stage_x_begin<WAVES, XLDS>(xr, x, M, K);
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (s_begin + u < s_end) issue(u, s_begin + u);
  stage_x_finish<WAVES, XLDS>(xr, x, xl, M, K);
  for (int base = s_begin; base < s_end; base += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int ks = base + u;
      if (ks < s_end) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          bf16x8 af;
          if constexpr (XLDS) af = xs_src.frag(mt, col, 32 * ks + 8 * kq);
          else af = a[u][mt];
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, b[u][nt], acc[mt][nt], 0, 0, 0);
        }
        if (ks + U < s_end) issue(u, ks + U);
      }
    }
  }
  gemv_epilogue<MT, NT, WAVES>(acc, red, y, M, N, nt0, ntiles);
}

// ---- launch plans -------------------------------------------------------------------------------
struct GemvPlan {
  int mt, nt, waves, u;
  bool xlds;
};

// Experiment hook (not part of the public interface): overrides nt / waves / u / xlds when >= 0.
int g_dbg_nt = -1, g_dbg_waves = -1, g_dbg_u = -1, g_dbg_xlds = -1;

constexpr int kXldsMaxBytes = 64 * 1024;

inline GemvPlan plan_gemv(int M, int N, int K, bool w4) {
  GemvPlan p;
  p.mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int ntiles = N >> 4;
  const int units = w4 ? (K >> 7) : (K >> 5);   // 1 KiB pieces per column tile
  // Measured on the 7B shapes: 2 pieces in flight per wave, 16 waves per workgroup for narrow
  // outputs (N <= 8192, one workgroup per CU), 8 otherwise; never fewer than u pieces per wave.
  p.nt = 1;
  p.u = w4 ? 2 : (p.mt == 1 ? 8 : 4);
  int waves = ntiles <= 512 ? 16 : 8;
  while (waves > 4 && units < waves * p.u) waves /= 2;
  p.waves = waves;
  p.xlds = p.mt == 1 && (int64_t)(M + 1) * K * 2 <= kXldsMaxBytes;
  if (g_dbg_nt >= 0) p.nt = g_dbg_nt;
  if (g_dbg_waves >= 0) p.waves = g_dbg_waves;
  if (g_dbg_u >= 0) p.u = g_dbg_u;
  if (g_dbg_xlds >= 0) p.xlds = g_dbg_xlds && p.mt == 1 && (int64_t)(M + 1) * K * 2 <= kXldsMaxBytes;
  return p;
}

template <typename Kern, typename... Args>
int launch_gemv(Kern kern, const GemvPlan& p, int M, int N, int K, hipStream_t stream, Args... args) {
  const size_t lds = (size_t)p.waves * p.mt * p.nt * 256 * 4 + (p.xlds ? (size_t)(M + 1) * K * 2 : 0);
  if (lds > 48 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return O355_ELAUNCH;
  const unsigned blocks = (unsigned)(((N >> 4) + p.nt - 1) / p.nt);
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(p.waves * 64), lds, stream, args..., M, N, K);
  O355_CHECK_LAUNCH();
}

}  // namespace

extern "C" void olmo355_debug_set_gemv_plan(int nt, int waves, int u, int xlds) {
  g_dbg_nt = nt, g_dbg_waves = waves, g_dbg_u = u, g_dbg_xlds = xlds;
}

#define W4_CASE(MTv, NTv, Wv, Uv, Xv)                                                                          \
  if (p.mt == MTv && p.nt == NTv && p.waves == Wv && p.u == Uv && p.xlds == Xv)                               \
    return launch_gemv(w4_gemv_kernel<MTv, NTv, Wv, Uv, Xv>, p, M, N, K, as_stream(stream), x, (const u32x4*)wt, st, zt, y);
#define B16_CASE(MTv, NTv, Wv, Uv, Xv)                                                                         \
  if (p.mt == MTv && p.nt == NTv && p.waves == Wv && p.u == Uv && p.xlds == Xv)                               \
    return launch_gemv(b16_gemv_kernel<MTv, NTv, Wv, Uv, Xv>, p, M, N, K, as_stream(stream), x, (const bf16x8*)wt, y);
#define FOR_WAVES(CASE, MTv, NTv, Uv, Xv) CASE(MTv, NTv, 4, Uv, Xv) CASE(MTv, NTv, 8, Uv, Xv) CASE(MTv, NTv, 16, Uv, Xv)

extern "C" int olmo355_w4_gemv(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                               uint16_t* y, int M, int N, int K, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (M > 64 || (K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  const GemvPlan p = plan_gemv(M, N, K, true);
  FOR_WAVES(W4_CASE, 1, 1, 4, true) FOR_WAVES(W4_CASE, 1, 1, 4, false)
  FOR_WAVES(W4_CASE, 1, 1, 2, true) FOR_WAVES(W4_CASE, 1, 1, 2, false)
  FOR_WAVES(W4_CASE, 1, 1, 8, true) FOR_WAVES(W4_CASE, 1, 2, 4, true) FOR_WAVES(W4_CASE, 1, 2, 2, true)
  FOR_WAVES(W4_CASE, 1, 4, 2, true) FOR_WAVES(W4_CASE, 1, 2, 2, false)
  FOR_WAVES(W4_CASE, 2, 1, 2, false) FOR_WAVES(W4_CASE, 4, 1, 2, false)
  return O355_EUNSUPPORTED;
}

extern "C" int olmo355_b16_gemv(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K,
                                void* stream) {
  if (!x || !wt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (M > 64 || (K & 31) || (N & 15)) return O355_EUNSUPPORTED;
  const GemvPlan p = plan_gemv(M, N, K, false);
  FOR_WAVES(B16_CASE, 1, 1, 8, true) FOR_WAVES(B16_CASE, 1, 1, 8, false)
  FOR_WAVES(B16_CASE, 1, 1, 4, true) FOR_WAVES(B16_CASE, 1, 2, 8, true) FOR_WAVES(B16_CASE, 1, 2, 4, true)
  FOR_WAVES(B16_CASE, 2, 1, 4, false) FOR_WAVES(B16_CASE, 4, 1, 4, false)
  return O355_EUNSUPPORTED;
}
