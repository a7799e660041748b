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
//
// Two optional fusions remove whole launches from a decode step (each launch costs several
// microseconds against kernels that themselves run for 5-10):
//   prologue  x := resid + rmsnorm(a; w, eps)   the post-norm residual update of the previous
//             sub-block (olmo/model.py:786-794,814-821), recomputed by every workgroup while
//             its first weight pieces are in flight; workgroup 0 also writes x to memory;
//   epilogue  y := silu(gate) * up              SwiGLU (olmo/model.py:365-368) on the two column
//             tiles a workgroup owns (tile p of the first half and tile p of the second half).
#include "common.h"

namespace {

struct GemvArgs {
  const uint16_t* x;       // [M,K] activations; with a prologue: the tensor to be normalised
  const uint16_t* resid;   // [M,K] residual stream (prologue) or null
  const uint16_t* norm_w;  // [K] RMSNorm weight (prologue) or null
  uint16_t* x_out;         // [M,K] resid + norm(x), written by workgroup 0 (prologue)
  uint16_t* y;             // [M,N], or [M,N/2] with the SwiGLU epilogue
  float eps;
  int M, N, K;
};

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

__device__ __forceinline__ void unpack8(const u32x4& v, float (&f)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) f[2 * i] = bf16lo_to_f32(v[i]), f[2 * i + 1] = bf16hi_to_f32(v[i]);
}

// ---- activation staging --------------------------------------------------------------------------
// XLDS: the M rows of x live in LDS as [M+1][K] (the extra row is zero and is what the padding
// lanes of the A operand read); every A fragment is one ds_read_b128 right before its MFMA.
// The global loads are issued in begin() -- before the weight prologue -- and consumed in
// finish(), after the weight loads have been issued; the barrier orders LDS only.
constexpr int kXStageRegs = 4;  // plain copy: 16-byte pieces per thread held across the weight prologue

template <int WAVES, bool XLDS, int PRO>
struct XStage {
  __device__ __forceinline__ void begin(const GemvArgs&) {}
  __device__ __forceinline__ void finish(const GemvArgs&, uint16_t*, float*) {}
};

template <int WAVES>
struct XStage<WAVES, true, 0> {
  u32x4 xr[kXStageRegs];
  __device__ __forceinline__ void begin(const GemvArgs& a) {
    const int total = (a.M * a.K) >> 3;
#pragma unroll
    for (int i = 0; i < kXStageRegs; ++i) {
      const int idx = threadIdx.x + i * WAVES * 64;
      if (idx < total) xr[i] = reinterpret_cast<const u32x4*>(a.x)[idx];
    }
  }
  __device__ __forceinline__ void finish(const GemvArgs& a, uint16_t* xl, float*) {
    const int total = (a.M * a.K) >> 3;
#pragma unroll
    for (int i = 0; i < kXStageRegs; ++i) {
      const int idx = threadIdx.x + i * WAVES * 64;
      if (idx < total) reinterpret_cast<u32x4*>(xl)[idx] = xr[i];
    }
    for (int idx = threadIdx.x + kXStageRegs * WAVES * 64; idx < total; idx += WAVES * 64)
      reinterpret_cast<u32x4*>(xl)[idx] = reinterpret_cast<const u32x4*>(a.x)[idx];
    for (int i = threadIdx.x; i < (a.K >> 3); i += WAVES * 64)
      reinterpret_cast<u32x4*>(xl + (int64_t)a.M * a.K)[i] = u32x4{0u, 0u, 0u, 0u};
    lds_barrier();
  }
};

// x := resid + w * round(a * rsqrt(mean(a^2) + eps)), rounding points of olmo/model.py:241-255 and
// of the bf16 residual add.  The whole workgroup shares the rows: thread t owns the 16-byte pieces
// t, t + threads, ... (VPT of them), a wave's 64 pieces lie in one row (K % 512 == 0), the per-wave
// sums of squares meet in LDS and are added in a fixed order.
template <int WAVES, int VPT>
struct NormStage {
  u32x4 av[VPT], rv[VPT], wv[VPT];
  __device__ __forceinline__ void begin(const GemvArgs& a) {
    const int nvec = a.K >> 3, total = a.M * nvec;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int idx = threadIdx.x + i * WAVES * 64;
      if (idx < total) {
        av[i] = reinterpret_cast<const u32x4*>(a.x)[idx];
        rv[i] = reinterpret_cast<const u32x4*>(a.resid)[idx];
        wv[i] = reinterpret_cast<const u32x4*>(a.norm_w)[idx % nvec];
      }
    }
  }
  __device__ __forceinline__ void finish(const GemvArgs& a, uint16_t* xl, float* part /* [VPT*WAVES] */) {
    const int nvec = a.K >> 3, total = a.M * nvec;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      float ss = 0.f;
      if (threadIdx.x + i * WAVES * 64 < total) {
        float f[8];
        unpack8(av[i], f);
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
      }
      ss = wave_sum(ss);
      if (lane == 0) part[i * WAVES + wave] = ss;
    }
    lds_barrier();
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int idx = threadIdx.x + i * WAVES * 64;
      if (idx < total) {
        const int m = idx / nvec;
        float ss = 0.f;  // partials of row m, in (i, wave) order
        for (int j = 0; j < VPT * WAVES; ++j) {
          const int first = (j % WAVES) * 64 + (j / WAVES) * WAVES * 64;  // first piece of that partial
          if (first < total && first / nvec == m) ss += part[j];
        }
        const float rstd = 1.f / sqrtf(ss / (float)a.K + a.eps);
        float f[8], r[8], w[8];
        unpack8(av[i], f);
        unpack8(rv[i], r);
        unpack8(wv[i], w);
        u32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float y0 = round_bf16(w[2 * e] * round_bf16(f[2 * e] * rstd));
          const float y1 = round_bf16(w[2 * e + 1] * round_bf16(f[2 * e + 1] * rstd));
          o[e] = pack_bf16x2(r[2 * e] + y0, r[2 * e + 1] + y1);
        }
        reinterpret_cast<u32x4*>(xl)[idx] = o;
        if (blockIdx.x == 0) reinterpret_cast<u32x4*>(a.x_out)[idx] = o;
      }
    }
    for (int i = threadIdx.x; i < nvec; i += WAVES * 64)
      reinterpret_cast<u32x4*>(xl + (int64_t)a.M * a.K)[i] = u32x4{0u, 0u, 0u, 0u};
    lds_barrier();
  }
};
template <int WAVES>
struct XStage<WAVES, true, 1> : NormStage<WAVES, 1> {};
template <int WAVES>
struct XStage<WAVES, true, 4> : NormStage<WAVES, 4> {};

// ---- epilogue: reduce over the waves in fixed order, write y (bf16) -----------------------------------
template <int MT, int NT, int WAVES, int EPI>
__device__ __forceinline__ void gemv_epilogue(f32x4 (&acc)[MT][NT], float* red, const GemvArgs& a,
                                              const int (&tile)[NT], int ntiles) {
  constexpr int PER_WAVE = MT * NT * 256;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave * PER_WAVE + ((mt * NT + nt) * 4 + r) * 64 + lane] = acc[mt][nt][r];
  __syncthreads();
  if constexpr (EPI == 0) {
    for (int i = threadIdx.x; i < PER_WAVE; i += WAVES * 64) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) v += red[w * PER_WAVE + i];
      const int l = i & 63, r = (i >> 6) & 3, t = i >> 8;
      const int nt = t % NT, mt = t / NT;
      const int m = mt * 16 + 4 * (l >> 4) + r;
      if (tile[nt] < ntiles && m < a.M) a.y[(int64_t)m * a.N + tile[nt] * 16 + (l & 15)] = f32_to_bf16_bits(v);
    }
  } else {
    static_assert(EPI == 0 || NT == 2, "the SwiGLU epilogue owns one up tile and one gate tile");
    const int half_n = a.N >> 1;
    for (int i = threadIdx.x; i < MT * 256; i += WAVES * 64) {
      const int l = i & 63, r = (i >> 6) & 3, mt = i >> 8;
      const int iu = ((mt * 2 + 0) * 4 + r) * 64 + l, ig = ((mt * 2 + 1) * 4 + r) * 64 + l;
      float up = 0.f, gate = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) up += red[w * PER_WAVE + iu], gate += red[w * PER_WAVE + ig];
      up = round_bf16(up), gate = round_bf16(gate);  // the Linear's bf16 output
      const float s = round_bf16(gate / (1.f + expf(-gate)));
      const int m = mt * 16 + 4 * (l >> 4) + r;
      if (m < a.M) a.y[(int64_t)m * half_n + tile[0] * 16 + (l & 15)] = f32_to_bf16_bits(s * up);
    }
  }
}

template <int NT, int EPI>
__device__ __forceinline__ void owned_tiles(int (&tile)[NT], int ntiles) {
  if constexpr (EPI == 1) {
    tile[0] = blockIdx.x;
    tile[1] = blockIdx.x + (ntiles >> 1);
  } else {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) tile[nt] = blockIdx.x * NT + nt;
  }
}

// ---- int4 -----------------------------------------------------------------------------------------------
template <int MT, int NT, int WAVES, int U, bool XLDS, int PRO, int EPI>
__global__ __launch_bounds__(WAVES * 64) void w4_gemv_kernel(GemvArgs args, const u32x4* __restrict__ wt,
                                                             const uint16_t* __restrict__ st,
                                                             const uint8_t* __restrict__ zt) {
  static_assert(!XLDS || MT == 1, "x in LDS is for M <= 16");
  static_assert(PRO == 0 || XLDS, "the norm prologue writes x into LDS");
  extern __shared__ __align__(16) unsigned char smem[];
  float* red = reinterpret_cast<float*>(smem);                                                // [WAVES][MT*NT*256]
  uint16_t* xl = reinterpret_cast<uint16_t*>(smem + WAVES * MT * NT * 256 * sizeof(float));   // [M+1][K]
  const int M = args.M, K = args.K;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kq = lane >> 4;
  const int G = K >> 7, ntiles = args.N >> 4;
  int tile[NT];
  owned_tiles<NT, EPI>(tile, ntiles);
  // contiguous slice of groups per wave
  const int g_begin = (int)((int64_t)G * wave / WAVES), g_end = (int)((int64_t)G * (wave + 1) / WAVES);
  const bf16x8 ones = ones_bf16x8();
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const uint16_t* xrow = xl + (col < M ? col : M) * K;  // this lane's row in LDS (XLDS)

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
      const int tnt = min(tile[nt], ntiles - 1);  // out-of-range tiles are computed and dropped
      const int64_t t = (int64_t)tnt * G + g;
      w[u][nt] = __builtin_nontemporal_load(&wt[t * 64 + lane]);
      s16[u][nt] = st[t * 16 + col];
      z8[u][nt] = zt[t * 8 + (col >> 1)];
    }
    if constexpr (!XLDS) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) a[u][j][mt] = load_x_frag(args.x, mt * 16 + col, M, K, 128 * g + 32 * j + 8 * kq);
    }
  };

  // x first (it comes from L2 and is needed first), then U weight pieces in flight
  XStage<WAVES, XLDS, PRO> stage;
  stage.begin(args);
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (g_begin + u < g_end) issue(u, g_begin + u);
  stage.finish(args, xl, red);

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
            if constexpr (XLDS) af[mt] = *reinterpret_cast<const bf16x8*>(xrow + 128 * g + 32 * j + 8 * kq);
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
  gemv_epilogue<MT, NT, WAVES, EPI>(acc, red, args, tile, ntiles);
}

// ---- dense bf16 --------------------------------------------------------------------------------------------
template <int MT, int NT, int WAVES, int U, bool XLDS, int PRO, int EPI>
__global__ __launch_bounds__(WAVES * 64) void b16_gemv_kernel(GemvArgs args, const bf16x8* __restrict__ wt) {
  static_assert(!XLDS || MT == 1, "x in LDS is for M <= 16");
  static_assert(PRO == 0 || XLDS, "the norm prologue writes x into LDS");
  extern __shared__ __align__(16) unsigned char smem[];
  float* red = reinterpret_cast<float*>(smem);
  uint16_t* xl = reinterpret_cast<uint16_t*>(smem + WAVES * MT * NT * 256 * sizeof(float));
  const int M = args.M, K = args.K;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kq = lane >> 4;
  const int KS = K >> 5, ntiles = args.N >> 4;
  int tile[NT];
  owned_tiles<NT, EPI>(tile, ntiles);
  const int s_begin = (int)((int64_t)KS * wave / WAVES), s_end = (int)((int64_t)KS * (wave + 1) / WAVES);
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const uint16_t* xrow = xl + (col < M ? col : M) * K;
  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = zero4;
  bf16x8 b[U][NT], a[XLDS ? 1 : U][MT];
  auto issue = [&](int u, int ks) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int tnt = min(tile[nt], ntiles - 1);
      b[u][nt] = __builtin_nontemporal_load(&wt[((int64_t)tnt * KS + ks) * 64 + lane]);
    }
    if constexpr (!XLDS) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) a[u][mt] = load_x_frag(args.x, mt * 16 + col, M, K, 32 * ks + 8 * kq);
    }
  };
  XStage<WAVES, XLDS, PRO> stage;
  stage.begin(args);
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (s_begin + u < s_end) issue(u, s_begin + u);
  stage.finish(args, xl, red);
  for (int base = s_begin; base < s_end; base += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int ks = base + u;
      if (ks < s_end) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          bf16x8 af;
          if constexpr (XLDS) af = *reinterpret_cast<const bf16x8*>(xrow + 32 * ks + 8 * kq);
          else af = a[u][mt];
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, b[u][nt], acc[mt][nt], 0, 0, 0);
        }
        if (ks + U < s_end) issue(u, ks + U);
      }
    }
  }
  gemv_epilogue<MT, NT, WAVES, EPI>(acc, red, args, tile, ntiles);
}

// ---- launch plans -------------------------------------------------------------------------------
struct GemvPlan {
  int mt, nt, waves;
  bool xlds;
  int pro, epi;
};

// Experiment hook (not part of the public interface): overrides waves / xlds when >= 0.
int g_dbg_waves = -1, g_dbg_xlds = -1;

constexpr int kXldsMaxBytes = 64 * 1024;

// u (pieces in flight per wave) is fixed per format: 2 KiB-groups for int4, 8 (4 for M > 16) 32-row steps for bf16
inline GemvPlan plan_gemv(int M, int N, int K, bool w4, bool pro, bool epi) {
  GemvPlan p;
  p.mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  p.nt = epi ? 2 : 1;
  p.pro = pro, p.epi = epi;
  const int ntiles = N >> 4;
  const int units = w4 ? (K >> 7) : (K >> 5);  // 1 KiB pieces per column tile
  const int u = w4 ? 2 : (p.mt == 1 ? 8 : 4);
  // Measured on the 7B shapes: 16 waves per workgroup for narrow outputs (N <= 8192, one workgroup
  // per CU), 8 otherwise; never fewer than u pieces per wave.
  int waves = ntiles <= 512 ? 16 : 8;
  while (waves > 4 && units < waves * u) waves /= 2;
  if (p.mt > 1 && waves > 8) waves = 8;  // register budget of the wider accumulators
  if (pro) {  // rows shared by the whole workgroup: 1 or 4 pieces per thread
    const int pieces = M * (K >> 3);
    if (pieces > waves * 64 && waves < 16 && units >= 16 * u) waves = 16;
    p.pro = pieces <= waves * 64 ? 1 : (pieces <= 4 * waves * 64 ? 4 : -1);
  }
  p.waves = waves;
  p.xlds = p.mt == 1 && (int64_t)(M + 1) * K * 2 <= kXldsMaxBytes;
  if (g_dbg_waves >= 0 && !pro && !epi) p.waves = g_dbg_waves;
  if (g_dbg_xlds >= 0 && !pro && !epi) p.xlds = g_dbg_xlds && p.xlds;
  return p;
}

template <typename Kern, typename... Args>
int launch_gemv(Kern kern, const GemvPlan& p, const GemvArgs& a, hipStream_t stream, Args... args) {
  const size_t lds = (size_t)p.waves * p.mt * p.nt * 256 * 4 + (p.xlds ? (size_t)(a.M + 1) * a.K * 2 : 0);
  if (lds > 48 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return O355_ELAUNCH;
  const int ntiles = a.N >> 4;
  const unsigned blocks = p.epi ? (unsigned)(ntiles >> 1) : (unsigned)((ntiles + p.nt - 1) / p.nt);
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(p.waves * 64), lds, stream, a, args...);
  O355_CHECK_LAUNCH();
}

int check_fused(const GemvArgs& a, bool pro, bool epi) {
  if (pro && (!a.resid || !a.norm_w || !a.x_out || a.M > 16 || (a.K & 511))) return O355_EUNSUPPORTED;
  if ((pro || epi) && (int64_t)(a.M + 1) * a.K * 2 > kXldsMaxBytes) return O355_EUNSUPPORTED;
  if (epi && ((a.N & 31) || a.M > 16)) return O355_EUNSUPPORTED;
  return O355_OK;
}

#define GEMV_CASE(KERNEL, MTv, NTv, Wv, Uv, Xv, Pv, Ev, ...)                                                  \
  if (p.mt == MTv && p.nt == NTv && p.waves == Wv && p.xlds == Xv && p.pro == Pv && p.epi == Ev)             \
    return launch_gemv(KERNEL<MTv, NTv, Wv, Uv, Xv, Pv, Ev>, p, a, as_stream(stream), __VA_ARGS__);
#define GEMV_WAVES(KERNEL, MTv, NTv, Uv, Xv, Pv, Ev, ...)        \
  GEMV_CASE(KERNEL, MTv, NTv, 4, Uv, Xv, Pv, Ev, __VA_ARGS__)    \
  GEMV_CASE(KERNEL, MTv, NTv, 8, Uv, Xv, Pv, Ev, __VA_ARGS__)    \
  GEMV_CASE(KERNEL, MTv, NTv, 16, Uv, Xv, Pv, Ev, __VA_ARGS__)

int w4_gemv_dispatch(const GemvArgs& a, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, bool pro, bool epi,
                     void* stream) {
  const GemvPlan p = plan_gemv(a.M, a.N, a.K, true, pro, epi);
  const u32x4* w = (const u32x4*)wt;
  GEMV_WAVES(w4_gemv_kernel, 1, 1, 2, true, 0, 0, w, st, zt)
  GEMV_WAVES(w4_gemv_kernel, 1, 1, 2, false, 0, 0, w, st, zt)
  GEMV_WAVES(w4_gemv_kernel, 2, 1, 2, false, 0, 0, w, st, zt)
  GEMV_WAVES(w4_gemv_kernel, 4, 1, 2, false, 0, 0, w, st, zt)
  GEMV_WAVES(w4_gemv_kernel, 1, 1, 2, true, 1, 0, w, st, zt)
  GEMV_WAVES(w4_gemv_kernel, 1, 1, 2, true, 4, 0, w, st, zt)
  GEMV_WAVES(w4_gemv_kernel, 1, 2, 2, true, 0, 1, w, st, zt)
  GEMV_WAVES(w4_gemv_kernel, 1, 2, 2, true, 1, 1, w, st, zt)
  GEMV_WAVES(w4_gemv_kernel, 1, 2, 2, true, 4, 1, w, st, zt)
  return O355_EUNSUPPORTED;
}

int b16_gemv_dispatch(const GemvArgs& a, const uint16_t* wt, bool pro, bool epi, void* stream) {
  const GemvPlan p = plan_gemv(a.M, a.N, a.K, false, pro, epi);
  const bf16x8* w = (const bf16x8*)wt;
  GEMV_WAVES(b16_gemv_kernel, 1, 1, 8, true, 0, 0, w)
  GEMV_WAVES(b16_gemv_kernel, 1, 1, 8, false, 0, 0, w)
  GEMV_WAVES(b16_gemv_kernel, 2, 1, 4, false, 0, 0, w)
  GEMV_WAVES(b16_gemv_kernel, 4, 1, 4, false, 0, 0, w)
  GEMV_WAVES(b16_gemv_kernel, 1, 1, 8, true, 1, 0, w)
  GEMV_WAVES(b16_gemv_kernel, 1, 1, 8, true, 4, 0, w)
  GEMV_WAVES(b16_gemv_kernel, 1, 2, 8, true, 0, 1, w)
  GEMV_WAVES(b16_gemv_kernel, 1, 2, 8, true, 1, 1, w)
  GEMV_WAVES(b16_gemv_kernel, 1, 2, 8, true, 4, 1, w)
  return O355_EUNSUPPORTED;
}

}  // namespace

extern "C" void olmo355_debug_set_gemv_plan(int waves, int xlds) { g_dbg_waves = waves, g_dbg_xlds = xlds; }

extern "C" int olmo355_w4_gemv(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                               uint16_t* y, int M, int N, int K, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (M > 64 || (K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  const GemvArgs a{x, nullptr, nullptr, nullptr, y, 0.f, M, N, K};
  return w4_gemv_dispatch(a, wt, st, zt, false, false, stream);
}

extern "C" int olmo355_b16_gemv(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K,
                                void* stream) {
  if (!x || !wt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (M > 64 || (K & 31) || (N & 15)) return O355_EUNSUPPORTED;
  const GemvArgs a{x, nullptr, nullptr, nullptr, y, 0.f, M, N, K};
  return b16_gemv_dispatch(a, wt, false, false, stream);
}

extern "C" int olmo355_w4_gemv_fused(const uint16_t* x, const uint16_t* resid, const uint16_t* norm_w, float eps,
                                     uint16_t* x_out, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                                     uint16_t* y, int M, int N, int K, int swiglu, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (M > 64 || (K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  const GemvArgs a{x, resid, norm_w, x_out, y, eps, M, N, K};
  const bool pro = resid != nullptr, epi = swiglu != 0;
  const int chk = check_fused(a, pro, epi);
  if (chk != O355_OK) return chk;
  return w4_gemv_dispatch(a, wt, st, zt, pro, epi, stream);
}

extern "C" int olmo355_b16_gemv_fused(const uint16_t* x, const uint16_t* resid, const uint16_t* norm_w, float eps,
                                      uint16_t* x_out, const uint16_t* wt, uint16_t* y, int M, int N, int K, int swiglu,
                                      void* stream) {
  if (!x || !wt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (M > 64 || (K & 31) || (N & 15)) return O355_EUNSUPPORTED;
  const GemvArgs a{x, resid, norm_w, x_out, y, eps, M, N, K};
  const bool pro = resid != nullptr, epi = swiglu != 0;
  const int chk = check_fused(a, pro, epi);
  if (chk != O355_OK) return chk;
  return b16_gemv_dispatch(a, wt, pro, epi, stream);
}
