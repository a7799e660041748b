// Small-M int4 / bf16 linear layers (decode): y[M,N] = x[M,K] . W[K,N], bandwidth-bound.  This file holds the
// kernels that keep all rows of x in LDS (or registers) per workgroup -- the lean kernel of the decode step
// (M <= 16, with the norm / SwiGLU fusions) and its older forms -- and the dispatcher of olmo355_w4_gemv*;
// plain products with 5..64 rows mostly go to gemv_mid.hip (see w4_gemv_dispatch).
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
#include <algorithm>

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
  // chained norms: the launch that produced x left the sum of squares of each 16-column tile of its
  // (bf16-rounded) output rows in ssq_in[M][K/16]; this launch leaves its own in ssq_out[M][N/16]
  const float* ssq_in = nullptr;
  float* ssq_out = nullptr;
};

__device__ __forceinline__ bf16x8 load_x_frag(const uint16_t* __restrict__ x, int row, int M, int K, int k) {
  if (row < M) return *reinterpret_cast<const bf16x8*>(x + (int64_t)row * K + k);
  u32x4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, z);
}

// ---- activation staging --------------------------------------------------------------------------
// XLDS: the M rows of x live in LDS as [M+1][K] (the extra row is zero and is what the padding
// lanes of the A operand read); every A fragment is one ds_read_b128 right before its MFMA.
// The global loads are issued in begin() -- before the weight prologue -- and consumed in
// finish(), after the weight loads have been issued; the barrier orders LDS only.
constexpr int kXStageRegs = 4;  // plain copy: 16-byte pieces per thread held across the weight prologue

// Per-group sums of the staged activations, xs[g][rp] (rp rows per group, row m of group g): 16
// consecutive 16-byte pieces are one group of 128, i.e. one row of 16 lanes.  `v` is the piece as
// it went into LDS; all 64 lanes call this, `valid` per lane (whole rows of lanes are valid or not).
__device__ __forceinline__ void group_sum_to_lds(const u32x4& v, bool valid, int idx, int nvec, float* xs, int rp) {
  float f[8], s = 0.f;
  unpack8(v, f);
#pragma unroll
  for (int e = 0; e < 8; ++e) s += f[e];
  s = row16_sum(valid ? s : 0.f);
  if (valid && (threadIdx.x & 15) == 0) xs[((idx % nvec) >> 4) * rp + idx / nvec] = s;
}

template <int WAVES, bool XLDS, int PRO>
struct XStage {
  __device__ __forceinline__ void begin(const GemvArgs&) {}
  template <bool XSUM = false>
  __device__ __forceinline__ void finish(const GemvArgs&, uint16_t*, float*, float* = nullptr, int = 0) {}
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
  template <bool XSUM = false>
  __device__ __forceinline__ void finish(const GemvArgs& a, uint16_t* xl, float*, float* xs = nullptr, int rp = 0) {
    const int total = (a.M * a.K) >> 3, nvec = a.K >> 3;
#pragma unroll
    for (int i = 0; i < kXStageRegs; ++i) {
      const int idx = threadIdx.x + i * WAVES * 64;
      if (idx < total) reinterpret_cast<u32x4*>(xl)[idx] = xr[i];
      if constexpr (XSUM) group_sum_to_lds(xr[i], idx < total, idx, nvec, xs, rp);
    }
    for (int idx = threadIdx.x + kXStageRegs * WAVES * 64; idx < total; idx += WAVES * 64) {
      const u32x4 v = reinterpret_cast<const u32x4*>(a.x)[idx];
      reinterpret_cast<u32x4*>(xl)[idx] = v;
      if constexpr (XSUM) group_sum_to_lds(v, true, idx, nvec, xs, rp);
    }
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
  template <bool XSUM = false>
  __device__ __forceinline__ void finish(const GemvArgs& a, uint16_t* xl, float* part /* [VPT*WAVES] */, float* xs = nullptr,
                                         int rp = 0) {
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
    u32x4 ov[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      ov[i] = u32x4{0u, 0u, 0u, 0u};
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
        ov[i] = o;
      }
    }
    if constexpr (XSUM) {
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int idx = threadIdx.x + i * WAVES * 64;
        group_sum_to_lds(ov[i], idx < total, idx, nvec, xs, rp);
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
  const UnpackConsts uc;
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
            const bf16x8 b = unpack_w4_bias128(w[u][nt][j], uc);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              t[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[mt], b, t[mt][nt], 0, 0, 0);
          }
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const float sc = (float)__builtin_bit_cast(_Float16, s16[u][nt]);
          const float nzc = -(float)(129 + (int)((z8[u][nt] >> (4 * (col & 1))) & 15u));  // -(128 + (stored + 1))
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
              acc[mt][nt][r] = __builtin_fmaf(sc, __builtin_fmaf(nzc, xsum[mt][r], t[mt][nt][r]), acc[mt][nt][r]);
        }
        if (g + U < g_end) issue(u, g + U);  // refill the slot just consumed
      }
    }
  }
  gemv_epilogue<MT, NT, WAVES, EPI>(acc, red, args, tile, ntiles);
}

// ---- int4, M <= 16: several groups share one accumulator --------------------------------------------------
// With M <= 4 only rows 0..3 of the 16-row MFMA tile carry data.  GPA = 4 consecutive groups of 128
// rows then use the *same* accumulator: group u of the four puts its activations in operand rows
// 4u..4u+3, so its products land in the lanes of row block u (lane = 16 u + column) while the other
// row blocks receive zeros.  The lanes of block u hold the scale and zero of group u, the sums of
// the activations per group come from LDS (computed once while staging), and the fp32 correction
// acc += scale * (T - (128 + zero) * X) is applied once per four groups instead of once per group.
// M <= 8 shares an accumulator between GPA = 2 groups; M <= 16 (GPA = 1) is the plain scheme.
template <int GPA, int NT, int WAVES, int PRO, int EPI>
__global__ __launch_bounds__(WAVES * 64) void w4_gemv_rot_kernel(GemvArgs args, const u32x4* __restrict__ wt,
                                                                 const uint16_t* __restrict__ st,
                                                                 const uint8_t* __restrict__ zt) {
  constexpr int RP = 16 / GPA;   // operand rows per group
  constexpr int KQS = 4 / GPA;   // lane row blocks (kq) per group
  extern __shared__ __align__(16) unsigned char smem[];
  const int M = args.M, K = args.K;
  const int G = K >> 7, ntiles = args.N >> 4;
  float* red = reinterpret_cast<float*>(smem);                                           // [WAVES][NT*256]
  uint16_t* xl = reinterpret_cast<uint16_t*>(smem + WAVES * NT * 256 * sizeof(float));   // [M+1][K]
  float* xs = reinterpret_cast<float*>(xl + (int64_t)(M + 1) * K);                       // [G][RP]
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int ul = kq / KQS;  // the group (of the GPA) whose results this lane holds
  int tile[NT];
  owned_tiles<NT, EPI>(tile, ntiles);
  const int g_begin = (int)((int64_t)G * wave / WAVES), g_end = (int)((int64_t)G * (wave + 1) / WAVES);
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const UnpackConsts uc;

  // operand row `col` of group slot u is activation row col - u*RP when that is in [0, M), else zeros
  int xoff[GPA];
#pragma unroll
  for (int u = 0; u < GPA; ++u) {
    const int rel = col - u * RP;
    xoff[u] = ((rel >= 0 && rel < M) ? rel : M) * K + 8 * kq;
  }

  f32x4 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt] = zero4;
  u32x4 w[GPA][NT];
  uint32_t s16c[NT], z8c[NT], s16n[NT], z8n[NT];
  int64_t tbase[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) tbase[nt] = (int64_t)min(tile[nt], ntiles - 1) * G;  // out-of-range tiles: computed, dropped

  auto issue_w = [&](int u, int g) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) w[u][nt] = __builtin_nontemporal_load(&wt[(tbase[nt] + g) * 64 + lane]);
  };
  auto issue_sz = [&](uint32_t (&s16)[NT], uint32_t (&z8)[NT], int base) {
    const int g = max(min(base + ul, g_end - 1), 0);  // a wave without groups still reads valid memory
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      s16[nt] = st[(tbase[nt] + g) * 16 + col];
      z8[nt] = zt[(tbase[nt] + g) * 8 + (col >> 1)];
    }
  };

  XStage<WAVES, true, PRO> stage;
  stage.begin(args);
#pragma unroll
  for (int u = 0; u < GPA; ++u)
    if (g_begin + u < g_end) issue_w(u, g_begin + u);
  issue_sz(s16c, z8c, g_begin);
  stage.template finish<true>(args, xl, red, xs, RP);

  for (int base = g_begin; base < g_end; base += GPA) {
    const bool more = base + GPA < g_end;
    if (more) issue_sz(s16n, z8n, base + GPA);
    f32x4 t[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) t[nt] = zero4;
#pragma unroll
    for (int u = 0; u < GPA; ++u) {
      const int g = base + u;
      if (g < g_end) {
        const uint16_t* xp = xl + xoff[u] + 128 * g;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bf16x8 af = *reinterpret_cast<const bf16x8*>(xp + 32 * j);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            t[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, unpack_w4_bias128(w[u][nt][j], uc), t[nt], 0, 0, 0);
        }
        if (g + GPA < g_end) issue_w(u, g + GPA);  // refill the slot just consumed
      }
    }
    // correction for this lane's group
    const int gl = base + ul;
    const f32x4 xg = *reinterpret_cast<const f32x4*>(xs + min(gl, g_end - 1) * RP + (4 * kq) % RP);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const float sc = gl < g_end ? (float)__builtin_bit_cast(_Float16, (uint16_t)s16c[nt]) : 0.f;
      const float nzc = -(float)(129 + (int)((z8c[nt] >> (4 * (col & 1))) & 15u));  // -(128 + (stored + 1))
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[nt][r] = __builtin_fmaf(sc, __builtin_fmaf(nzc, xg[r], t[nt][r]), acc[nt][r]);
    }
    if (more) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) s16c[nt] = s16n[nt], z8c[nt] = z8n[nt];
    }
  }

  // ---- reduce over waves and over the GPA row blocks, in fixed order ---------------------------------
  constexpr int PER_WAVE = NT * 256;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave * PER_WAVE + (nt * 4 + r) * 64 + lane] = acc[nt][r];
  __syncthreads();
  // output element (m = 4 kqs + r, column c) of tile nt: lanes c + 16 (u KQS + kqs), u = 0..GPA-1
  auto total_of = [&](int nt, int r, int kqs, int c) {
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv)
#pragma unroll
      for (int u = 0; u < GPA; ++u) v += red[wv * PER_WAVE + (nt * 4 + r) * 64 + c + 16 * (u * KQS + kqs)];
    return v;
  };
  if constexpr (EPI == 0) {
    for (int i = threadIdx.x; i < NT * RP * 16; i += WAVES * 64) {
      const int c = i & 15, m = (i >> 4) % RP, nt = i / (16 * RP);
      if (tile[nt] < ntiles && m < M)
        args.y[(int64_t)m * args.N + tile[nt] * 16 + c] = f32_to_bf16_bits(total_of(nt, m & 3, m >> 2, c));
    }
  } else {
    static_assert(EPI == 0 || NT == 2, "the SwiGLU epilogue owns one up tile and one gate tile");
    const int half_n = args.N >> 1;
    for (int i = threadIdx.x; i < RP * 16; i += WAVES * 64) {
      const int c = i & 15, m = i >> 4;
      if (m < M) {
        const float up = round_bf16(total_of(0, m & 3, m >> 2, c));  // the Linear's bf16 output
        const float gate = round_bf16(total_of(1, m & 3, m >> 2, c));
        const float sg = round_bf16(gate / (1.f + expf(-gate)));
        args.y[(int64_t)m * half_n + tile[0] * 16 + c] = f32_to_bf16_bits(sg * up);
      }
    }
  }
}

// ---- norm prologue for M <= 4 ---------------------------------------------------------------------------
// Same arithmetic and rounding points as NormStage, written for few instructions: buffer loads
// with the thread index as offset, rows found by comparison instead of division (M <= 4 and a wave's
// 64 pieces lie in one row, K % 512 == 0), sums over a wave with DPP.
template <int WAVES, int VPT>
struct SmallNorm {
  u32x4 av[VPT], rv[VPT], wv[VPT];
  int row[VPT];  // row of this wave's pieces in pass i (wave-uniform), -1 past the end
  __device__ __forceinline__ void begin(const GemvArgs& a, int wave) {
    const int nvec = a.K >> 3, total = a.M * nvec;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(a.x, (int64_t)total * 16), rr = make_rsrc(a.resid, (int64_t)total * 16),
                                 rn = make_rsrc(a.norm_w, (int64_t)nvec * 16);
    const int voff = (threadIdx.x & 63) * 16;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int past = (wave + i * WAVES) * 64;  // first piece of this wave in pass i
      const int first = min(past, total - 64);   // past the end: re-read the last pieces (nvec is a multiple of 64), unused
      const int m = (first >= nvec) + (first >= 2 * nvec) + (first >= 3 * nvec);
      row[i] = past < total ? m : -1;
      av[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, voff, first * 16, 0));
      rv[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rr, voff, first * 16, 0));
      wv[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rn, voff, (first - m * nvec) * 16, 0));
    }
  }
  // part: [VPT*WAVES] floats of LDS
  __device__ __forceinline__ void finish(const GemvArgs& a, uint16_t* xl, float* part, int wave) {
    const int nvec = a.K >> 3, total = a.M * nvec;
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      float f[8], ss = 0.f;
      unpack8(av[i], f);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
      ss = wave_sum_dpp(ss);
      if (lane == 0) part[i * WAVES + wave] = ss;
    }
    lds_barrier();
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      if (row[i] >= 0) {  // wave-uniform
        float ss = 0.f;   // partials of this row, in (pass, wave) order
#pragma unroll
        for (int j = 0; j < VPT * WAVES; ++j) {
          const int first = ((j % WAVES) + (j / WAVES) * WAVES) * 64;
          const int mj = (first >= nvec) + (first >= 2 * nvec) + (first >= 3 * nvec);
          if (first < total && mj == row[i]) ss += part[j];
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
        const int idx = (wave + i * WAVES) * 64 + lane;
        reinterpret_cast<u32x4*>(xl)[idx] = o;
        if (blockIdx.x == 0) reinterpret_cast<u32x4*>(a.x_out)[idx] = o;
      }
    }
    for (int i = threadIdx.x; i < nvec; i += WAVES * 64)
      reinterpret_cast<u32x4*>(xl + (int64_t)a.M * a.K)[i] = u32x4{0u, 0u, 0u, 0u};
    lds_barrier();
  }
};

// ---- norm prologue fed by the producer's sums of squares --------------------------------------------------
// mean(a^2) of a row is the sum of K/16 per-tile partials that the launch which wrote `a` left behind,
// so a wave needs no other wave: it adds the partials (fixed order: lane-strided, then the DPP tree),
// normalises just its own slice of the row and goes on without a workgroup barrier.
constexpr int kChainPieces = 4;  // at most: 16-byte pieces per lane = rows x KiB of slice

template <int P>  // pieces per lane (1, 2 or 4); also bounds the rows
struct ChainNorm {
  u32x4 av[P], rv[P], wv[P];
  f32x4 pv[P][4];  // partial sums: row, chunk of 256
  __device__ __forceinline__ static void piece_of(int p, int per_row, int& m, int& k) {
    m = per_row == 1 ? p : (per_row == 2 ? p >> 1 : (per_row == 3 ? p / 3 : p >> 2));
    k = p - m * per_row;
  }
  // lo, hi: byte range of the wave's slice within a row
  __device__ __forceinline__ void begin(const GemvArgs& a, int lo, int hi) {
    const int lane = threadIdx.x & 63, n_ssq = a.K >> 4, per_row = (hi - lo + 1023) >> 10;
#pragma unroll
    for (int m = 0; m < P; ++m) {
      const __amdgpu_buffer_rsrc_t rp = make_rsrc(a.ssq_in + (int64_t)min(m, a.M - 1) * n_ssq, (int64_t)n_ssq * 4);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        pv[m][c] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (m < a.M && c * 256 < n_ssq)
          pv[m][c] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rp, lane * 16, c * 1024, 0));
      }
    }
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(a.x, (int64_t)a.M * a.K * 2), rr = make_rsrc(a.resid, (int64_t)a.M * a.K * 2),
                                 rn = make_rsrc(a.norm_w, (int64_t)a.K * 2);
#pragma unroll
    for (int p = 0; p < P; ++p) {
      int m, k;
      piece_of(p, per_row, m, k);
      if (m < a.M) {  // wave-uniform
        const int off = lo + k * 1024;
        av[p] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, lane * 16, m * a.K * 2 + off, 0));
        rv[p] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rr, lane * 16, m * a.K * 2 + off, 0));
        wv[p] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rn, lane * 16, off, 0));
      }
    }
  }
  __device__ __forceinline__ void finish(const GemvArgs& a, unsigned char* smem, int lo, int hi) {
    const int lane = threadIdx.x & 63, per_row = (hi - lo + 1023) >> 10;
    const int n_ssq = a.K >> 4;
    float rstd[P];
#pragma unroll
    for (int m = 0; m < P; ++m) {
      rstd[m] = 0.f;
      if (m < a.M) {  // wave-uniform
        float ss = (pv[m][0][0] + pv[m][0][1]) + (pv[m][0][2] + pv[m][0][3]);
#pragma unroll
        for (int c = 1; c < 4; ++c)
          if (c * 256 < n_ssq) ss += (pv[m][c][0] + pv[m][c][1]) + (pv[m][c][2] + pv[m][c][3]);
        ss = wave_sum_dpp(ss);
        rstd[m] = 1.f / sqrtf(ss / (float)a.K + a.eps);
      }
    }
#pragma unroll
    for (int p = 0; p < P; ++p) {
      int m, k;
      piece_of(p, per_row, m, k);
      if (m < a.M) {
        const int off = lo + k * 1024 + lane * 16;
        float rs = rstd[0];
#pragma unroll
        for (int q = 1; q < P; ++q) rs = m == q ? rstd[q] : rs;
        float f[8], r[8], w[8];
        unpack8(av[p], f);
        unpack8(rv[p], r);
        unpack8(wv[p], w);
        u32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float y0 = round_bf16(w[2 * e] * round_bf16(f[2 * e] * rs));
          const float y1 = round_bf16(w[2 * e + 1] * round_bf16(f[2 * e + 1] * rs));
          o[e] = pack_bf16x2(r[2 * e] + y0, r[2 * e + 1] + y1);
        }
        if (off < hi) {  // lanes past the slice would mix rows
          *reinterpret_cast<u32x4*>(smem + m * a.K * 2 + off) = o;
          if (blockIdx.x == 0) *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(a.x_out) + m * a.K * 2 + off) = o;
        }
      }
    }
  }
};

// ---- int4, M <= 4: the lean decode kernel ---------------------------------------------------------------
// A decode launch lives for a few microseconds and every SIMD interleaves several waves, so each
// instruction of the per-wave preamble costs (waves per SIMD) x 4 cycles before the first weight
// request leaves.  This variant keeps the preamble short: buffer loads with scalar offsets (no
// per-lane 64-bit address arithmetic), the activations copied memory -> LDS directly (no registers,
// no VALU), all weight requests of the wave issued before anything else is waited for, the sums of
// the activations from the matrix cores (B = ones) instead of a staging pass.  GPA = 4, 2 or 1 groups
// share an accumulator as in w4_gemv_rot_kernel (M <= 4, 8, 16); the norm prologues exist for GPA = 4.
// F16 (plain products only): fp16 activations and output on the fp16 matrix instruction.  The weights are then what
// the reference's QuantLinear multiplies with, fp16(scale * (q - zero)), formed per word before the product (no sums
// of the activations, no correction afterwards): every lane also fetches scale and zero of its own column for each
// group in flight.
template <int GPA, int NT, int WAVES, int PRO, int EPI, bool F16 = false>
__device__ __forceinline__ void w4_gemv_small_body(const GemvArgs& args, const u32x4* __restrict__ wt,
                                                   const uint16_t* __restrict__ st, const uint8_t* __restrict__ zt) {
  constexpr int RP = 16 / GPA;  // operand rows per group slot
  constexpr int KQS = 4 / GPA;  // lane row blocks per slot
  static_assert(PRO == 0 || GPA == 4, "the norm prologues are written for M <= 4");
  static_assert(!F16 || (PRO == 0 && EPI == 0), "fp16 activations: plain products");
  extern __shared__ __align__(16) unsigned char smem[];
  const int M = args.M, K = args.K;
  const int G = K >> 7, ntiles = args.N >> 4, nvec = K >> 3;
  const int xbytes = M * K * 2;
  // LDS: x rows [M][K], a zero row [K], then the reduction area
  const int red_off = xbytes + max(K * 2, 1024);  // a direct copy may run up to 1 KiB past the rows (zeros)
  uint16_t* xl = reinterpret_cast<uint16_t*>(smem);
  float* red = reinterpret_cast<float*>(smem + red_off);  // [WAVES][NT][RP rows][16 columns]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int g_begin = (G * wave) / WAVES, g_end = (G * (wave + 1)) / WAVES;
  int tile[NT], tg[NT];
  owned_tiles<NT, EPI>(tile, ntiles);
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) tg[nt] = min(tile[nt], ntiles - 1) * G;  // out-of-range tiles: computed, dropped

  const __amdgpu_buffer_rsrc_t rw = make_rsrc(wt, (int64_t)ntiles * G * 1024);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(st, (int64_t)ntiles * G * 32);
  const __amdgpu_buffer_rsrc_t rz = make_rsrc(zt, (int64_t)ntiles * G * 8);
  const int ul = kq / KQS;  // the slot whose results this lane holds
  const int wvoff = lane * 16, svoff = (ul * 16 + col) * 2, zvoff = ul * 8 + (col >> 1);

  u32x4 w[GPA][NT];
  uint32_t s16c[NT], z8c[NT], s16n[NT], z8n[NT];
  // slot u of a quad is group base+u, clamped into the matrix so that every request is valid and
  // the number of requests per wave is fixed
  auto issue_w = [&](int u, int g) {
    const int gc = min(g, G - 1);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      w[u][nt] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, wvoff, (tg[nt] + gc) * 1024, 2));
  };
  // the lanes of slot ul hold the scale and zero of group base+ul: one contiguous request each
  auto issue_sz = [&](uint32_t (&s16)[NT], uint32_t (&z8)[NT], int base) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      s16[nt] = __builtin_amdgcn_raw_buffer_load_b16(rs, svoff, (tg[nt] + base) * 32, 0);
      z8[nt] = __builtin_amdgcn_raw_buffer_load_b8(rz, zvoff, (tg[nt] + base) * 8, 0);
    }
  };

  // ---- activations first (they are needed first and come from L2), then the whole first quad ----
  // Without a norm prologue every wave stages just the columns of x it will multiply (its own
  // groups), so no workgroup barrier is needed before the main loop.
  int n_x = 0;  // direct-to-LDS requests of this wave (wave-uniform)
  if constexpr (PRO == 0) {
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(args.x, xbytes);
    const int lo = g_begin * 256, hi = g_end * 256;  // byte range of the wave's slice within a row
    for (int m = 0; m < M; ++m)
      for (int off = lo; off < hi; off += 1024) {
        // lanes past the slice (or the row) read past the buffer or into the next wave's slice: harmless,
        // the LDS rows are laid out like memory and neighbours write the same bytes
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)(smem + m * K * 2 + off), 16, wvoff, m * K * 2 + off, 0, 0);
        ++n_x;
      }
  }
  constexpr bool CHAIN = PRO >= 8;  // 8, 9, 10: chained norm with 1, 2, 4 pieces per lane
  SmallNorm<WAVES, (PRO == 0 || CHAIN) ? 1 : PRO> norm;
  ChainNorm<CHAIN ? (1 << (PRO - 8)) : 1> chain;
  if constexpr (CHAIN) chain.begin(args, g_begin * 256, g_end * 256);
  else if constexpr (PRO != 0) norm.begin(args, wave);
  uint32_t sq[F16 ? GPA : 1][NT], zq[F16 ? GPA : 1][NT];  // F16: scale and zero of (group in slot u, this lane's column)
  auto issue_szq = [&](int u, int g) {
    const int gc = min(g, G - 1);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      sq[F16 ? u : 0][nt] = __builtin_amdgcn_raw_buffer_load_b16(rs, col * 2, (tg[nt] + gc) * 32, 0);
      zq[F16 ? u : 0][nt] = __builtin_amdgcn_raw_buffer_load_b8(rz, col >> 1, (tg[nt] + gc) * 8, 0);
    }
  };
#pragma unroll
  for (int u = 0; u < GPA; ++u) issue_w(u, g_begin + u);
  if constexpr (F16) {
#pragma unroll
    for (int u = 0; u < GPA; ++u) issue_szq(u, g_begin + u);
  } else {
    issue_sz(s16c, z8c, g_begin);
  }
  if constexpr (PRO == 0 || CHAIN) {
    // zero row, this wave's slice of it
    for (int off = g_begin * 256 + lane * 16; off < g_end * 256; off += 1024)
      *reinterpret_cast<u32x4*>(smem + xbytes + off) = u32x4{0u, 0u, 0u, 0u};
    if constexpr (CHAIN) chain.finish(args, smem, g_begin * 256, g_end * 256);
    // everything but the GPA*NT weight and 2*NT scale/zero requests has arrived: the slice is in LDS
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(F16 ? 3 * GPA * NT : GPA * NT + 2 * NT, true));
  } else {
    norm.finish(args, xl, red, wave);
  }

  // operand row `col` of slot u is activation row col - u*RP when that is in [0, M), else the zero row
  int xoff[GPA];
#pragma unroll
  for (int u = 0; u < GPA; ++u) {
    const int rel = col - RP * u;
    xoff[u] = ((rel >= 0 && rel < M) ? rel : M) * K + 8 * kq;
  }
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const bf16x8 ones = ones_bf16x8();
  const UnpackConsts uc;
  auto mma = [](const bf16x8& a_, const bf16x8& b_, const f32x4& c_) {
    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    if constexpr (F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a_), __builtin_bit_cast(f16x8, b_), c_, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_, b_, c_, 0, 0, 0);
  };
  f32x4 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt] = zero4;

  if constexpr (F16) {
    for (int base = g_begin; base < g_end; base += GPA) {
#pragma unroll
      for (int u = 0; u < GPA; ++u) {
        const int g = base + u;
        if (g < g_end) {
          const uint16_t* xp = xl + xoff[u] + 128 * g;
          DequantConstsF16 dc[NT];
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            dc[nt] = dequant_consts_f16((uint16_t)sq[u][nt], 1 + (int)((zq[u][nt] >> (4 * (col & 1))) & 15u));  // stored zero points are one less
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const bf16x8 af = *reinterpret_cast<const bf16x8*>(xp + 32 * j);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
              acc[nt] = mma(af, __builtin_bit_cast(bf16x8, dequant_word_f16(w[u][nt][j], dc[nt])), acc[nt]);
          }
          if (g + GPA < g_end) {  // refill the slot just consumed
            issue_w(u, g + GPA);
            issue_szq(u, g + GPA);
          }
        }
      }
    }
  }
  for (int base = g_begin; !F16 && base < g_end; base += GPA) {
    const bool more = base + GPA < g_end;
    if (more) issue_sz(s16n, z8n, base + GPA);
    f32x4 t[NT], xsum = zero4;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) t[nt] = zero4;
#pragma unroll
    for (int u = 0; u < GPA; ++u) {
      const int g = base + u;
      if (g < g_end) {
        const uint16_t* xp = xl + xoff[u] + 128 * g;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bf16x8 af = *reinterpret_cast<const bf16x8*>(xp + 32 * j);
          xsum = mma(af, ones, xsum);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) t[nt] = mma(af, unpack_w4_bias128(w[u][nt][j], uc), t[nt]);
        }
        if (g + GPA < g_end) issue_w(u, g + GPA);  // refill the slot just consumed
      }
    }
    // fp32 correction; rows of a slot whose group lies past the wave's range are all zero
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const float sc = (float)__builtin_bit_cast(_Float16, (uint16_t)s16c[nt]);
      const float nzc = -(float)(129 + (int)((z8c[nt] >> (4 * (col & 1))) & 15u));  // -(128 + (stored + 1))
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[nt][r] = __builtin_fmaf(sc, __builtin_fmaf(nzc, xsum[r], t[nt][r]), acc[nt][r]);
    }
    if (more) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) s16c[nt] = s16n[nt], z8c[nt] = z8n[nt];
    }
  }

  // ---- reduce: the slots inside the wave, then the waves through LDS, in fixed order ----------------
  // this lane's rows are m = 4 (kq % KQS) + r; lanes kq and kq + KQS, ... hold the other slots' shares
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (GPA == 4 && r >= M) continue;  // rows past M hold nothing (uniform: with GPA = 4 a lane's rows are r)
      float v = acc[nt][r];
      if constexpr (GPA == 4) v = combine_xor16(v, AddOp{});
      if constexpr (GPA >= 2) v = combine_xor32(v, AddOp{});
      if (kq < KQS) red[((wave * NT + nt) * RP + 4 * kq + r) * 16 + col] = v;
    }
  __syncthreads();
  auto total_of = [&](int nt, int m, int c) {
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) v += red[((wv * NT + nt) * RP + m) * 16 + c];
    return v;
  };
  if constexpr (EPI == 0) {
    for (int i = tid; i < NT * RP * 16; i += WAVES * 64) {  // whole waves: 16 lanes = one (row, tile)
      const int c = i & 15, m = (i >> 4) % RP, nt = (i >> 4) / RP;
      const bool live = tile[nt] < ntiles && m < M;
      float v = 0.f;
      if constexpr (F16) {
        const _Float16 hv = (_Float16)(live ? total_of(nt, m, c) : 0.f);
        v = (float)hv;
        if (live) args.y[(int64_t)m * args.N + tile[nt] * 16 + c] = __builtin_bit_cast(uint16_t, hv);
      } else {
        v = live ? round_bf16(total_of(nt, m, c)) : 0.f;
        if (live) args.y[(int64_t)m * args.N + tile[nt] * 16 + c] = f32_to_bf16_bits(v);
      }
      if (args.ssq_out) {  // sum of squares of the 16 outputs of (row, tile): one row of 16 lanes
        const float q = row16_sum(v * v);
        if (live && c == 0) args.ssq_out[(int64_t)m * ntiles + tile[nt]] = q;
      }
    }
  } else {
    static_assert(EPI == 0 || NT == 2, "the SwiGLU epilogue owns one up tile and one gate tile");
    if (tid < RP * 16) {
      const int c = tid & 15, m = tid >> 4;
      if (m < M) {
        const float up = round_bf16(total_of(0, m, c));  // the Linear's bf16 output
        const float gate = round_bf16(total_of(1, m, c));
        const float sg = round_bf16(gate / (1.f + expf(-gate)));
        args.y[(int64_t)m * (args.N >> 1) + tile[0] * 16 + c] = f32_to_bf16_bits(sg * up);
      }
    }
  }
}

template <int GPA, int NT, int WAVES, int PRO, int EPI, bool F16 = false>
__global__ __launch_bounds__(WAVES * 64) void w4_gemv_small_kernel(GemvArgs args, const u32x4* __restrict__ wt,
                                                                   const uint16_t* __restrict__ st,
                                                                   const uint8_t* __restrict__ zt) {
  w4_gemv_small_body<GPA, NT, WAVES, PRO, EPI, F16>(args, wt, st, zt);
}

// ---- int4, one row: the batch-1 decode step ----------------------------------------------------------------
// Time stamps inside w4_gemv_small_kernel at one row (the four linears of a 7B layer) showed a kernel bound by the
// number of instructions its waves issue, not by memory: six waves per SIMD of ~900 instructions each, the weights of
// a wave (4 KiB) already there when its activations are, a median wave 2.4 us into an 8 us launch before its own
// requests are out.  This kernel is the same product with the row count, the tile count per workgroup and the length
// of a wave's run of K fixed at compile time, so that what is left is close to what the format needs (per 16-byte
// piece of weights: four fragment reads, 28 unpack instructions, four matrix instructions):
//   * sizes come precomputed from the host (32-bit buffer ranges, group counts): no 64-bit clamps on the device;
//   * a wave's run of K is QUADS pieces of 1 KiB = QUADS x 4 groups; the row's pieces travel through registers in
//     either mode (copied, or normalised with the producer's sums of squares: ChainNorm's arithmetic), so the
//     compiler places every wait, and the per-group sums of the activations for the zero-point term are four
//     two-element dot products and a 16-lane sum on the piece a lane already holds (row i of 16 lanes = group i of the
//     quad = the accumulator rows of slot i);
//   * fragment reads address LDS with one base per slot and immediate offsets; every weight request of the wave is
//     issued before anything is waited for.
// Same accumulation order as the kernel above (groups in order inside a quad, quads in order, slots by the two
// half-wave exchanges, waves in order), same rounding points.
struct OneArgs {
  const uint16_t* x;       // [K] activations; with the prologue: the row to be normalised
  const uint16_t* resid;   // [K] residual stream (prologue)
  const uint16_t* norm_w;  // [K] RMSNorm weight (prologue)
  uint16_t* x_out;         // [K] resid + norm(x), written by workgroup 0 (prologue)
  const float* ssq_in;     // [K/16] per-tile sums of squares of x (prologue)
  const u32x4* wt;
  const uint16_t* st;
  const uint8_t* zt;
  uint16_t* y;             // [N], or [N/2] with the SwiGLU epilogue
  float* ssq_out;          // [N/16] or null
  float eps, k_float;
  int K, G, half_tiles;    // half_tiles: N/32 (SwiGLU: distance between an up tile and its gate tile)
  uint32_t wt_bytes, st_bytes, zt_bytes;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc32(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

// PRO: 0 plain; 1, 2: chained norm prologue with one or two 16-byte requests per lane for the sums of squares
// (K <= 4096, K <= 8192).  NG: groups of the wave with the longest run of K (every wave has NG or NG - 1).  NT column
// tiles per workgroup: consecutive ones, or with EPI 1 (SwiGLU) NT/2 consecutive up tiles and their gate tiles.  More
// tiles per workgroup = fewer workgroups that each read the whole row (and, with the prologue, the residual and the
// norm weight) out of L2: at N = 12288 those reads are as many bytes as the weights.
// Every wave issues the same requests in the same order (the compiler counts them to place its waits, and requests
// inside branches make it wait for everything): the one slot a shorter wave does not have is asked for past the end of
// the buffer, which answers with zeros and moves nothing.
template <int WAVES, int PRO, int EPI, int NG, int NT>
__global__ __launch_bounds__(WAVES * 64) void w4_gemv_one_kernel(OneArgs a) {
  static_assert(EPI == 0 || (NT & 1) == 0, "SwiGLU: tiles in (up, gate) pairs");
  constexpr int QUADS = (NG + 3) / 4;
  extern __shared__ __align__(16) unsigned char smem[];
  const int K2 = a.K * 2;  // LDS: the row, a row of zeros, [WAVES][NT][16] partial results
  float* red = reinterpret_cast<float*>(smem + 2 * K2);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int G = a.G;
  const int g_begin = (G * wave) / WAVES, g_end = (G * (wave + 1)) / WAVES;
  const bool full = g_end - g_begin == NG;  // else NG - 1 groups (the host checks)
  const int run = (g_end - g_begin) * 256;  // bytes of the wave's run of the row
  const int lo = g_begin * 256;             // where it starts
  int tg[NT];  // first group of tile nt in the tiled weights; EPI: nt = 2 pair + (0 up, 1 gate)
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    tg[nt] = (EPI ? (int)blockIdx.x * (NT / 2) + (nt >> 1) + (nt & 1) * a.half_tiles : (int)blockIdx.x * NT + nt) * G;
  const int wvoff = lane * 16;

  // ---- 1. the row's pieces (from L2: asked for first), then every weight request of the wave ------------
  // (a lane past the wave's run reads the neighbour's bytes, or zeros past the row, and is dropped below)
  u32x4 av[QUADS], rv[QUADS], nv[QUADS];
  f32x4 pv[PRO == 2 ? 2 : 1];
  {
    const __amdgpu_buffer_rsrc_t ra = make_rsrc32(a.x, (uint32_t)K2);
    if constexpr (PRO != 0) {
      const __amdgpu_buffer_rsrc_t rp = make_rsrc32(a.ssq_in, (uint32_t)(a.K >> 2));  // K/16 floats; zeros past the end
      pv[0] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rp, wvoff, 0, 0));
      if constexpr (PRO == 2) pv[1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rp, wvoff, 1024, 0));
    }
#pragma unroll
    for (int q = 0; q < QUADS; ++q)
      av[q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, wvoff, lo + q * 1024, 0));
    if constexpr (PRO != 0) {
      const __amdgpu_buffer_rsrc_t rr = make_rsrc32(a.resid, (uint32_t)K2), rn = make_rsrc32(a.norm_w, (uint32_t)K2);
#pragma unroll
      for (int q = 0; q < QUADS; ++q) {
        rv[q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rr, wvoff, lo + q * 1024, 0));
        nv[q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rn, wvoff, lo + q * 1024, 0));
      }
    }
  }
  u32x4 w[NG][NT];
  uint16_t s16[QUADS][NT];
  uint8_t z8[QUADS][NT];
  const __amdgpu_buffer_rsrc_t rw = make_rsrc32(a.wt, a.wt_bytes), rs = make_rsrc32(a.st, a.st_bytes), rz = make_rsrc32(a.zt, a.zt_bytes);
  const int svoff = (kq * 16 + col) * 2, zvoff = kq * 8 + (col >> 1);  // the lanes of slot kq: scale and zero of group kq of the quad
  const int last_voff = full ? wvoff : (int)0x80000000u;             // past every buffer: zeros, no traffic
  auto request = [&](int nt) {
#pragma unroll
    for (int g = 0; g < NG; ++g)
      w[g][nt] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, g == NG - 1 ? last_voff : wvoff, (tg[nt] + g_begin + g) * 1024, 2));
    // (groups past the wave's run: another group's finite numbers or the range check's zeros, times zero)
#pragma unroll
    for (int q = 0; q < QUADS; ++q) {
      s16[q][nt] = __builtin_amdgcn_raw_buffer_load_b16(rs, svoff, (tg[nt] + g_begin + 4 * q) * 32, 0);
      z8[q][nt] = __builtin_amdgcn_raw_buffer_load_b8(rz, zvoff, (tg[nt] + g_begin + 4 * q) * 8, 0);
    }
  };
  // (all of them ahead of the prologue: holding some back until the row is in LDS, which helps at eight rows, measured
  // level or slower here)
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) request(nt);
  // the wave's run of the zero row
#pragma unroll
  for (int q = 0; q < QUADS; ++q)
    if (q * 1024 + wvoff < run) *reinterpret_cast<u32x4*>(smem + K2 + lo + q * 1024 + wvoff) = u32x4{0u, 0u, 0u, 0u};

  // ---- 2. the row: normalised (ChainNorm's arithmetic and order of additions) or as it is, into LDS ---------
  float rstd = 0.f;
  if constexpr (PRO != 0) {
    float ss = (pv[0][0] + pv[0][1]) + (pv[0][2] + pv[0][3]);
    if constexpr (PRO == 2) ss += (pv[1][0] + pv[1][1]) + (pv[1][2] + pv[1][3]);
    ss = wave_sum_dpp(ss);
    rstd = 1.f / sqrtf(ss / a.k_float + a.eps);
  }
  typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
  const bf16x2v one2 = {(__bf16)1.f, (__bf16)1.f};
  float xsum[QUADS];  // of this lane's group (slot kq) of quad q
#pragma unroll
  for (int q = 0; q < QUADS; ++q) {
    u32x4 o = av[q];
    if constexpr (PRO != 0) {
      float f[8], r[8], wn[8];
      unpack8(av[q], f);
      unpack8(rv[q], r);
      unpack8(nv[q], wn);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float y0 = round_bf16(wn[2 * e] * round_bf16(f[2 * e] * rstd));
        const float y1 = round_bf16(wn[2 * e + 1] * round_bf16(f[2 * e + 1] * rstd));
        o[e] = pack_bf16x2(r[2 * e] + y0, r[2 * e + 1] + y1);
      }
    }
    const bool in = q * 1024 + wvoff < run;  // whole rows of 16 lanes
    if (in) {
      *reinterpret_cast<u32x4*>(smem + lo + q * 1024 + wvoff) = o;
      if constexpr (PRO != 0) {
        if (blockIdx.x == 0) *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(a.x_out) + lo + q * 1024 + wvoff) = o;
      }
    }
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) sum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2v, (uint32_t)o[e]), one2, sum, false);
    sum = row16_sum(sum);
    xsum[q] = in ? sum : 0.f;
  }

  // ---- 3. products.  Operand row `col` of slot u is the row itself for col == 4 u and zeros otherwise; a wave reads
  // only what it wrote ----------------------------------------------------------------------------------------
  const unsigned char* xb[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) xb[u] = smem + (col == 4 * u ? 0 : K2) + lo + 16 * kq;
  const UnpackConsts uc;
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  float acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt] = 0.f;
#pragma unroll
  for (int q = 0; q < QUADS; ++q) {
    f32x4 t[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) t[nt] = zero4;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int g = 4 * q + u;
      if (g < NG && (g < NG - 1 || full)) {  // compile-time but for the last slot (uniform)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bf16x8 af = *reinterpret_cast<const bf16x8*>(xb[u] + g * 256 + 64 * j);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            t[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, unpack_w4_bias128(w[g < NG ? g : 0][nt][j], uc), t[nt], 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const float sc = (float)__builtin_bit_cast(_Float16, s16[q][nt]);
      const float nzc = -(float)(129 + (int)(((uint32_t)z8[q][nt] >> (4 * (col & 1))) & 15u));  // -(128 + (stored + 1))
      acc[nt] = __builtin_fmaf(sc, __builtin_fmaf(nzc, xsum[q], t[nt][0]), acc[nt]);
    }
  }

  // ---- 4. the four slots of a wave, then the waves through LDS, in fixed order ---------------------------------
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    float v = combine_xor32(combine_xor16(acc[nt], AddOp{}), AddOp{});
    if (kq == 0) red[(wave * NT + nt) * 16 + col] = v;
  }
  __syncthreads();
  auto total_of = [&](int nt, int c) {
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) v += red[(wv * NT + nt) * 16 + c];
    return v;
  };
  if constexpr (EPI == 0) {
    if (tid < NT * 16) {  // whole rows of 16 lanes: one tile each
      const int c = tid & 15, tile = (int)blockIdx.x * NT + (tid >> 4);
      const float v = round_bf16(total_of(tid >> 4, c));
      a.y[tile * 16 + c] = f32_to_bf16_bits(v);
      if (a.ssq_out) {
        const float sq = row16_sum(v * v);
        if (c == 0) a.ssq_out[tile] = sq;
      }
    }
  } else {
    if (tid < (NT / 2) * 16) {
      const int c = tid & 15, p = tid >> 4;
      const float up = round_bf16(total_of(2 * p, c));  // the Linear's bf16 output
      const float gate = round_bf16(total_of(2 * p + 1, c));
      const float sg = round_bf16(gate / (1.f + expf(-gate)));
      a.y[((int)blockIdx.x * (NT / 2) + p) * 16 + c] = f32_to_bf16_bits(sg * up);
    }
  }
}

// ---- int4, 5 .. 8 rows: the activations as operand fragments, never whole in LDS ------------------------------
// With eight rows the two groups of 128 that share a matrix instruction fill its 16 operand rows exactly
// (rows 0-7: group g, rows 8-15: group g + 1), so a wave keeps the fragments of its own run of K in registers: no
// copy of all of x in LDS (eight rows of K = 11008 would not fit), no zero row, no barrier before the first product,
// and all of a wave's requests -- weights, scales, activations -- leave before anything is waited for.  The rows
// are asked for as they lie in memory (half a wave per row, 16 bytes per lane: a lane of the operand layout would ask
// for 16 bytes of a line of its own, and the texture path handles a quad of lanes at a time) and turned into
// fragments through 4 KiB of LDS that belong to the wave alone (written and read by the same wave, in order, so
// without a barrier; blocks of 256 bytes 272 apart, so that both the writes and the fragment reads touch every
// bank once).  The operand is shared by both groups, so group g's weights also multiply rows 8-15 (and the other way
// round): each group of the pair accumulates into registers of its own and a lane keeps the half that means
// something (rows 0-7 of the first, 8-15 of the second) when scale and zero are applied.  A workgroup owns NT
// column tiles (NT / 2 up-and-gate pairs with the SwiGLU epilogue) and all of K, split over its waves in runs of at
// most PMAX pairs of groups.
// PRO: the chained norm prologue x := resid + rmsnorm(a; w, eps): wave r adds up the sums of squares of row r
// and leaves 1 / rms in LDS (the one barrier, while everything else is in flight), and a lane normalises the pieces
// it has asked for before they go through LDS; workgroup 0 writes x_out.
constexpr int kR8BlockBytes = 272, kR8WaveBytes = 16 * kR8BlockBytes;

template <int NT, int PMAX>
struct R8Weights {  // one set of NT column tiles over a wave's run of K: packed pieces, scales, zeros as they arrive
  u32x4 w[PMAX][2][NT];
  uint32_t s16[PMAX][NT], z8[PMAX][NT];
};

// The grid stays (at most one workgroup per CU) and a workgroup walks the sets of NT tiles blockIdx.x,
// blockIdx.x + gridDim.x, ...: the fragments of x -- and with PRO the work of normalising them -- are paid for once
// per workgroup, not once per set, and the next set's weights are on their way while this one is multiplied.
// PF: with more sets than workgroups, ask for the next set's weights before this one is multiplied (a second
// set of registers); without it a workgroup still walks its sets, each waiting for its own requests.
template <int NT, int WAVES, int PMAX, bool PRO, int EPI, bool PF>
__global__ __launch_bounds__(WAVES * 64) void w4_gemv_r8_kernel(GemvArgs args, const u32x4* __restrict__ wt,
                                                                const uint16_t* __restrict__ st,
                                                                const uint8_t* __restrict__ zt) {
  static_assert(EPI == 0 || (NT & 1) == 0, "the SwiGLU epilogue owns up-and-gate pairs of tiles");
  extern __shared__ __align__(16) unsigned char smem[];
  float* red = reinterpret_cast<float*>(smem);  // [2][WAVES][NT][8 rows][16 columns]: sets alternate between the halves
  float* rstd_l = red + 2 * WAVES * NT * 128;   // [8]
  const int M = args.M, K = args.K;
  const int G = K >> 7, ntiles = args.N >> 4;
  const int n_sets = EPI == 1 ? ((ntiles >> 1) + NT / 2 - 1) / (NT / 2) : (ntiles + NT - 1) / NT;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  unsigned char* xs = smem + (2 * WAVES * NT * 128 + 8) * 4 + wave * kR8WaveBytes;  // this wave's own 16 blocks
  const int col = lane & 15, kq = lane >> 4;
  const int ul = kq >> 1;  // the group of a pair whose results this lane keeps
  const int g_begin = (G * wave) / WAVES, g_end = (G * (wave + 1)) / WAVES;
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(wt, (int64_t)ntiles * G * 1024);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(st, (int64_t)ntiles * G * 32);
  const __amdgpu_buffer_rsrc_t rz = make_rsrc(zt, (int64_t)ntiles * G * 8);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(args.x, (int64_t)M * K * 2);
  constexpr int kNowhere = 0x40000000;  // past every buffer here: such a request returns zeros
  const int wvoff = lane * 16;
  // as asked for: request i of a pair covers rows 2 i and 2 i + 1, a lane 16 bytes = 8 of the pair's 256 columns
  const int half = lane >> 5, c32 = lane & 31, cu = c32 >> 4;  // cu: which group of the pair the lane's columns lie in

  auto tile_of_set = [&](int set, int nt) {
    if constexpr (EPI == 1) return set * (NT / 2) + (nt >> 1) + ((nt & 1) ? (ntiles >> 1) : 0);
    else return set * NT + nt;
  };
  auto tile_live = [&](int set, int nt) {
    if constexpr (EPI == 1) return set * (NT / 2) + (nt >> 1) < (ntiles >> 1);
    else return set * NT + nt < ntiles;
  };
  auto request = [&](auto& r, int set) {
    int tg[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) tg[nt] = min(tile_of_set(set, nt), ntiles - 1) * G;  // out-of-range tiles: computed, dropped
#pragma unroll
    for (int p = 0; p < PMAX; ++p) {
      const int g = g_begin + 2 * p;
      if (g < g_end) {  // wave-uniform
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int gc = min(g + u, G - 1);  // a second group past the matrix: any valid piece, its rows of x are zero
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            r.w[p][u][nt] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, wvoff, (tg[nt] + gc) * 1024, 2));
        }
        // the lanes that keep group g + ul hold its scale and zero (zeros past the matrix: the range check looks at
        // the per-lane offset, so that is where "nowhere" has to stand)
        const int svoff = g + ul < G ? (ul * 16 + col) * 2 : kNowhere, zvoff = g + ul < G ? ul * 8 + (col >> 1) : kNowhere;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          r.s16[p][nt] = __builtin_amdgcn_raw_buffer_load_b16(rs, svoff, (tg[nt] + g) * 32, 0);
          r.z8[p][nt] = __builtin_amdgcn_raw_buffer_load_b8(rz, zvoff, (tg[nt] + g) * 8, 0);
        }
      }
    }
  };

  u32x4 xa[PMAX][4];  // first the rows as asked for (PRO: of the tensor to be normalised), then the operand fragments
  // rows past M lie past the buffer and read as zeros; so must the second group of a pair that reaches past the run
  auto x_voff = [&](int g) { return (g + cu < g_end) ? half * K * 2 + 256 * g + 16 * c32 : kNowhere; };
#pragma unroll
  for (int p = 0; p < PMAX; ++p) {
    const int g = g_begin + 2 * p;
    if (g < g_end) {
      const int xo = x_voff(g);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        xa[p][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, xo + 2 * i * K * 2, 0, 0));
    }
  }
  u32x4 xr[PRO ? PMAX : 1][4], xw[PRO ? PMAX : 1];
  f32x4 pv[4];
  if constexpr (PRO) {
    const __amdgpu_buffer_rsrc_t rr = make_rsrc(args.resid, (int64_t)M * K * 2), rn = make_rsrc(args.norm_w, (int64_t)K * 2);
    const int n_ssq = K >> 4;
    if (wave < M) {  // the sum of squares of row `wave`: n_ssq partials, lane-strided
      const __amdgpu_buffer_rsrc_t rp = make_rsrc(args.ssq_in + (int64_t)wave * n_ssq, (int64_t)n_ssq * 4);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        pv[c] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (c * 256 < n_ssq) pv[c] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rp, lane * 16, c * 1024, 0));
      }
    }
#pragma unroll
    for (int p = 0; p < PMAX; ++p) {
      const int g = g_begin + 2 * p;
      if (g < g_end) {
        const int xo = x_voff(g);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          xr[p][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rr, xo + 2 * i * K * 2, 0, 0));
        xw[p] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rn, (g + cu < g_end) ? 256 * g + 16 * c32 : kNowhere, 0, 0));
      }
    }
  }
  R8Weights<NT, PMAX> cur;
  R8Weights<NT, PF ? PMAX : 1> nxt;
  int set = blockIdx.x;
  if (set < n_sets) request(cur, set);

  if constexpr (PRO) {
    if (wave < M) {
      const int n_ssq = K >> 4;
      float ss = (pv[0][0] + pv[0][1]) + (pv[0][2] + pv[0][3]);
#pragma unroll
      for (int c = 1; c < 4; ++c)
        if (c * 256 < n_ssq) ss += (pv[c][0] + pv[c][1]) + (pv[c][2] + pv[c][3]);
      ss = wave_sum_dpp(ss);
      if (lane == 0) rstd_l[wave] = 1.f / sqrtf(ss / (float)K + args.eps);
    }
    __syncthreads();
    float rstd[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) rstd[i] = 2 * i + half < M ? rstd_l[2 * i + half] : 0.f;
#pragma unroll
    for (int p = 0; p < PMAX; ++p) {
      const int g = g_begin + 2 * p;
      if (g < g_end) {
        float wn[8];
        unpack8(xw[p], wn);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (2 * i >= M) continue;  // both rows of the request lie past M: zeros came back, zeros stay
          const int row = 2 * i + half;
          const bool mine = row < M && g + cu < g_end;
          float f[8], r[8];
          unpack8(xa[p][i], f);
          unpack8(xr[p][i], r);
          u32x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float y0 = round_bf16(wn[2 * e] * round_bf16(f[2 * e] * rstd[i]));
            const float y1 = round_bf16(wn[2 * e + 1] * round_bf16(f[2 * e + 1] * rstd[i]));
            o[e] = pack_bf16x2(r[2 * e] + y0, r[2 * e + 1] + y1);
          }
          xa[p][i] = mine ? o : u32x4{0u, 0u, 0u, 0u};
          if (blockIdx.x == 0 && mine)
            *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(args.x_out) + (int64_t)row * K * 2 + 256 * g + 16 * c32) = o;
        }
      }
    }
  }
  // rows as asked for -> operand fragments, a pair at a time through the wave's own blocks: block (row, group of the
  // pair) holds that row's 128 columns; the fragment of k-step j is chunk 4 j + kq of block (col & 7, col >> 3)
#pragma unroll
  for (int p = 0; p < PMAX; ++p) {
    const int g = g_begin + 2 * p;
    if (g < g_end) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<u32x4*>(xs + (2 * (2 * i + half) + cu) * kR8BlockBytes + (c32 & 15) * 16) = xa[p][i];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        xa[p][j] = *reinterpret_cast<const u32x4*>(xs + (2 * (col & 7) + (col >> 3)) * kR8BlockBytes + (4 * j + kq) * 16);
    }
  }

  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const bf16x8 ones = ones_bf16x8();
  const UnpackConsts uc;
  // the sums of the activations over each group do not depend on the tile: once, before the sets
  f32x4 xsum[PMAX];
#pragma unroll
  for (int p = 0; p < PMAX; ++p) {
    xsum[p] = zero4;
    if (g_begin + 2 * p < g_end) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        xsum[p] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[p][j]), ones, xsum[p], 0, 0, 0);
    }
  }
  int parity = 0;
  for (; set < n_sets; set += gridDim.x, parity ^= 1) {
    const int next = set + gridDim.x;
    if constexpr (PF) {
      if (next < n_sets) request(nxt, next);
    }
    f32x4 acc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] = zero4;
#pragma unroll
    for (int p = 0; p < PMAX; ++p) {
      const int g = g_begin + 2 * p;
      if (g < g_end) {
        f32x4 t[2][NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) t[0][nt] = zero4, t[1][nt] = zero4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bf16x8 af = __builtin_bit_cast(bf16x8, xa[p][j]);
#pragma unroll
          for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
              t[u][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, unpack_w4_bias128(cur.w[p][u][nt][j], uc), t[u][nt], 0, 0, 0);
        }
        // this lane's rows are 4 kq + r of the operand: group g for kq < 2, group g + 1 otherwise
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const float sc = (float)__builtin_bit_cast(_Float16, (uint16_t)cur.s16[p][nt]);
          const float nzc = -(float)(129 + (int)((cur.z8[p][nt] >> (4 * (col & 1))) & 15u));  // -(128 + (stored + 1))
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float tv = ul ? t[1][nt][r] : t[0][nt][r];
            acc[nt][r] = __builtin_fmaf(sc, __builtin_fmaf(nzc, xsum[p][r], tv), acc[nt][r]);
          }
        }
      }
    }
    // ---- reduce: the two groups of a pair inside the wave, then the waves through LDS, in fixed order ----------
    float* redp = red + parity * (WAVES * NT * 128);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float v = combine_xor32(acc[nt][r], AddOp{});
        if (kq < 2) redp[((wave * NT + nt) * 8 + 4 * kq + r) * 16 + col] = v;
      }
    __syncthreads();  // the only one per set: the next set writes the other half of `red`
    auto total_of = [&](int nt, int mm, int c) {
      float v = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) v += redp[((wv * NT + nt) * 8 + mm) * 16 + c];
      return v;
    };
    if constexpr (EPI == 0) {
      for (int i = tid; i < NT * 128; i += WAVES * 64) {  // whole waves: 16 lanes = one (row, tile)
        const int c = i & 15, mm = (i >> 4) & 7, nt = i >> 7;
        const int tl = tile_of_set(set, nt);
        const bool live = tile_live(set, nt) && mm < M;
        const float v = live ? round_bf16(total_of(nt, mm, c)) : 0.f;
        if (live) args.y[(int64_t)mm * args.N + tl * 16 + c] = f32_to_bf16_bits(v);
        if (args.ssq_out) {  // sum of squares of the 16 outputs of (row, tile): one row of 16 lanes
          const float q = row16_sum(v * v);
          if (live && c == 0) args.ssq_out[(int64_t)mm * ntiles + tl] = q;
        }
      }
    } else {
      for (int i = tid; i < (NT / 2) * 128; i += WAVES * 64) {
        const int c = i & 15, mm = (i >> 4) & 7, pr = i >> 7;
        if (mm < M && tile_live(set, 2 * pr)) {
          const float up = round_bf16(total_of(2 * pr, mm, c));  // the Linear's bf16 output
          const float gate = round_bf16(total_of(2 * pr + 1, mm, c));
          const float sg = round_bf16(gate / (1.f + expf(-gate)));
          args.y[(int64_t)mm * (args.N >> 1) + tile_of_set(set, 2 * pr) * 16 + c] = f32_to_bf16_bits(sg * up);
        }
      }
    }
    if (next < n_sets) {
      if constexpr (PF) cur = nxt;
      else request(cur, next);
    }
  }
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

// ---- int4, up to 8 rows, every request of a wave issued at once ------------------------------------------------------
// w4_gemv_r8_kernel's arithmetic (operand fragments of a wave's run of K in registers, two groups per matrix
// instruction, the same order of additions) in the shape that made the one-row kernel faster: the units of a workgroup
// (tiles, or up/gate pairs) are fixed at compile time and all asked for before anything is waited for, and every wave
// issues the same requests in the same order -- what a wave does not have (a group or a pair past its run, a unit past
// the last) is asked for past the end of the buffer -- so the compiler's own waits let the products of the first
// pieces start while the rest travels, where the requests inside branches of the kernel above made every wait a wait
// for everything.  One barrier for the reduction over the waves (one more with the prologue, for the rows' norms).
// PRO: 0, or the chained norm prologue with 1 or 2 requests per lane for a row's sums of squares (K <= 4096 / 8192).
// NP: pairs of groups of the wave with the longest run.  PER units per workgroup: b, b + gridDim.x, ...
template <int WAVES, int PRO, int EPI, int NP, int PER>
__global__ __launch_bounds__(WAVES * 64) void w4_gemv_rows_kernel(GemvArgs args, const u32x4* __restrict__ wt,
                                                                  const uint16_t* __restrict__ st,
                                                                  const uint8_t* __restrict__ zt, int units) {
  constexpr int NT = EPI ? 2 * PER : PER;  // tiles; EPI: nt = 2 unit + (0 up, 1 gate)
  extern __shared__ __align__(16) unsigned char smem[];
  float* red = reinterpret_cast<float*>(smem);  // [WAVES][NT][8 rows][16 columns]
  float* rstd_l = red + WAVES * NT * 128;       // [8]
  const int M = args.M, K = args.K;
  const int G = K >> 7, ntiles = args.N >> 4;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  unsigned char* xs = smem + (WAVES * NT * 128 + 8) * 4 + wave * kR8WaveBytes;  // this wave's own 16 blocks
  const int col = lane & 15, kq = lane >> 4;
  const int ul = kq >> 1;  // the group of a pair whose results this lane keeps
  const int g_begin = (G * wave) / WAVES, g_end = (G * (wave + 1)) / WAVES;
  constexpr int kNowhere = (int)0x80000000u;  // past every buffer: such a request returns zeros and moves nothing
  const int wvoff = lane * 16;
  const int half = lane >> 5, c32 = lane & 31, cu = c32 >> 4;  // request i of a pair: rows 2 i + half, group cu of the pair

  // ---- 1. the rows (from L2: first), then every weight request ------------------------------------------------------
  u32x4 xa[NP][4];  // first the rows as asked for (PRO: of the tensor to be normalised), then the operand fragments
  u32x4 xr[PRO ? NP : 1][4], xw[PRO ? NP : 1];
  f32x4 pv[PRO == 2 ? 2 : 1];
  {
    const __amdgpu_buffer_rsrc_t rx = make_rsrc32(args.x, (uint32_t)(M * K * 2));
    if constexpr (PRO != 0) {  // the sum of squares of row `wave` (waves past M: of the last row, unused)
      const int n_ssq = K >> 4;
      const __amdgpu_buffer_rsrc_t rp = make_rsrc32(args.ssq_in + min(wave, M - 1) * n_ssq, (uint32_t)(n_ssq * 4));
      pv[0] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rp, wvoff, 0, 0));
      if constexpr (PRO == 2) pv[1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rp, wvoff, 1024, 0));
    }
    // rows past M lie past the buffer and read as zeros; so must the second group of a pair that reaches past the run
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int g = g_begin + 2 * p;
      const int xo = (g + cu < g_end) ? half * K * 2 + 256 * g + 16 * c32 : kNowhere;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        xa[p][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, xo + 2 * i * K * 2, 0, 0));
    }
    if constexpr (PRO != 0) {
      const __amdgpu_buffer_rsrc_t rr = make_rsrc32(args.resid, (uint32_t)(M * K * 2)), rn = make_rsrc32(args.norm_w, (uint32_t)(K * 2));
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        const int g = g_begin + 2 * p;
        const bool in = g + cu < g_end;
        const int xo = in ? half * K * 2 + 256 * g + 16 * c32 : kNowhere;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          xr[p][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rr, xo + 2 * i * K * 2, 0, 0));
        xw[p] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rn, in ? 256 * g + 16 * c32 : kNowhere, 0, 0));
      }
    }
  }
  u32x4 w[NT][NP][2];
  uint16_t s16[NT][NP];
  uint8_t z8[NT][NP];
  const uint32_t n_groups = (uint32_t)ntiles * (uint32_t)G;
  const __amdgpu_buffer_rsrc_t rw = make_rsrc32(wt, n_groups * 1024u), rs = make_rsrc32(st, n_groups * 32u), rz = make_rsrc32(zt, n_groups * 8u);
  auto request = [&](int nt) {
    const int un = (int)blockIdx.x + (EPI ? nt >> 1 : nt) * (int)gridDim.x;
    const bool have = un < units;  // uniform
    const int tg = (EPI ? un + (nt & 1) * (ntiles >> 1) : un) * G;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int g = g_begin + 2 * p;
#pragma unroll
      for (int u = 0; u < 2; ++u)  // a group past the run: nothing is moved, and its rows of x are zero
        w[nt][p][u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, have && g + u < g_end ? wvoff : kNowhere, (tg + g + u) * 1024, 2));
      // the lanes that keep group g + ul hold its scale and zero
      const bool real = have && g + ul < g_end;
      s16[nt][p] = __builtin_amdgcn_raw_buffer_load_b16(rs, real ? (ul * 16 + col) * 2 : kNowhere, (tg + g) * 32, 0);
      z8[nt][p] = __builtin_amdgcn_raw_buffer_load_b8(rz, real ? ul * 8 + (col >> 1) : kNowhere, (tg + g) * 8, 0);
    }
  };
  // With the prologue only the first unit's weights are asked for ahead of it and the others after it (measured at
  // eight rows, att_proj / ff_proj of the 7B model: 10.7 / 15.2 us; two units ahead 12.0 / 16.2, all three 12.4 /
  // 17.6; the others asked for right after the norms' barrier, before the rows are normalised, 11.5 / 16.1): the
  // prologue is what such a launch waits for, and a CU's whole share of the weights in flight holds it back.
  constexpr int AHEAD = PRO != 0 ? (EPI ? 2 : 1) : NT;
#pragma unroll
  for (int nt = 0; nt < AHEAD; ++nt) request(nt);
  __builtin_amdgcn_sched_barrier(0);

  // ---- 2. the rows: normalised in place (ChainNorm's arithmetic), then turned into operand fragments -------------------
  if constexpr (PRO != 0) {
    float ss = (pv[0][0] + pv[0][1]) + (pv[0][2] + pv[0][3]);
    if constexpr (PRO == 2) ss += (pv[1][0] + pv[1][1]) + (pv[1][2] + pv[1][3]);
    ss = wave_sum_dpp(ss);
    if (lane == 0 && wave < 8) rstd_l[wave] = 1.f / sqrtf(ss / (float)K + args.eps);
    __syncthreads();
    float rstd[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) rstd[i] = rstd_l[2 * i + half];  // rows past M: some finite number, dropped below
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int g = g_begin + 2 * p;
      float wn[8];
      unpack8(xw[p], wn);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (2 * i >= M) continue;  // both rows of the request lie past M: zeros came back, zeros stay (uniform)
        const int row = 2 * i + half;
        const bool mine = row < M && g + cu < g_end;
        float f[8], r[8];
        unpack8(xa[p][i], f);
        unpack8(xr[p][i], r);
        u32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float y0 = round_bf16(wn[2 * e] * round_bf16(f[2 * e] * rstd[i]));
          const float y1 = round_bf16(wn[2 * e + 1] * round_bf16(f[2 * e + 1] * rstd[i]));
          o[e] = pack_bf16x2(r[2 * e] + y0, r[2 * e + 1] + y1);
        }
        xa[p][i] = mine ? o : u32x4{0u, 0u, 0u, 0u};
        if (blockIdx.x == 0 && mine)
          *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(args.x_out) + row * K * 2 + 256 * g + 16 * c32) = o;
      }
    }
  }
  // rows as asked for -> operand fragments, a pair at a time through the wave's own blocks: block (row, group of the
  // pair) holds that row's 128 columns; the fragment of k-step j is chunk 4 j + kq of block (col & 7, col >> 3)
#pragma unroll
  for (int p = 0; p < NP; ++p) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<u32x4*>(xs + (2 * (2 * i + half) + cu) * kR8BlockBytes + (c32 & 15) * 16) = xa[p][i];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      xa[p][j] = *reinterpret_cast<const u32x4*>(xs + (2 * (col & 7) + (col >> 3)) * kR8BlockBytes + (4 * j + kq) * 16);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int nt = AHEAD; nt < NT; ++nt) request(nt);
  __builtin_amdgcn_sched_barrier(0);
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const bf16x8 ones = ones_bf16x8();
  const UnpackConsts uc;
  f32x4 xsum[NP];  // the sums of the activations over each group do not depend on the tile
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    xsum[p] = zero4;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      xsum[p] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[p][j]), ones, xsum[p], 0, 0, 0);
  }

  // ---- 3. products, tile by tile in the order the pieces were asked for ------------------------------------------------
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    f32x4 acc = zero4;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      f32x4 t[2] = {zero4, zero4};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bf16x8 af = __builtin_bit_cast(bf16x8, xa[p][j]);
#pragma unroll
        for (int u = 0; u < 2; ++u)
          t[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, unpack_w4_bias128(w[nt][p][u][j], uc), t[u], 0, 0, 0);
      }
      // this lane's rows are 4 kq + r of the operand: group g for kq < 2, group g + 1 otherwise
      const float sc = (float)__builtin_bit_cast(_Float16, s16[nt][p]);
      const float nzc = -(float)(129 + (int)(((uint32_t)z8[nt][p] >> (4 * (col & 1))) & 15u));  // -(128 + (stored + 1))
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float tv = ul ? t[1][r] : t[0][r];
        acc[r] = __builtin_fmaf(sc, __builtin_fmaf(nzc, xsum[p][r], tv), acc[r]);
      }
    }
    // the two groups of a pair inside the wave; the waves through LDS below
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float v = combine_xor32(acc[r], AddOp{});
      if (kq < 2) red[((wave * NT + nt) * 8 + 4 * kq + r) * 16 + col] = v;
    }
  }
  __syncthreads();
  auto total_of = [&](int nt, int mm, int c) {
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) v += red[((wv * NT + nt) * 8 + mm) * 16 + c];
    return v;
  };
  for (int i = tid; i < PER * 128; i += WAVES * 64) {  // whole waves: 16 lanes = one (row, unit)
    const int c = i & 15, mm = (i >> 4) & 7, iu = i >> 7;
    const int un = (int)blockIdx.x + iu * (int)gridDim.x;
    const bool live = un < units && mm < M;
    if constexpr (EPI == 0) {
      const float v = live ? round_bf16(total_of(iu, mm, c)) : 0.f;
      if (live) args.y[mm * args.N + un * 16 + c] = f32_to_bf16_bits(v);
      if (args.ssq_out) {  // sum of squares of the 16 outputs of (row, tile): one row of 16 lanes
        const float q = row16_sum(v * v);
        if (live && c == 0) args.ssq_out[mm * ntiles + un] = q;
      }
    } else if (live) {
      const float up = round_bf16(total_of(2 * iu, mm, c));  // the Linear's bf16 output
      const float gate = round_bf16(total_of(2 * iu + 1, mm, c));
      const float sg = round_bf16(gate / (1.f + expf(-gate)));
      args.y[mm * (args.N >> 1) + un * 16 + c] = f32_to_bf16_bits(sg * up);
    }
  }
}

// ---- launch plans -------------------------------------------------------------------------------
struct GemvPlan {
  int mt, nt, waves;
  bool xlds;
  int pro, epi;
};

// Which kernel family a plain product goes to (olmo355_w4_gemv_form; 0 for every other entry point)
enum GemvForm { kFormChoose = 0, kFormLean = 1, kFormMid = 2, kFormMid1 = 3, kFormMid2 = 4, kFormOlder = 5 };

constexpr int kXldsMaxBytes = 64 * 1024;     // activations (+ zero row) in LDS, kernels for M <= 16
constexpr int kSmallMaxBytes = 128 * 1024;   // the same for the lean M <= 4 kernel (160 KiB of LDS per CU)

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
  if ((pro || epi) && (int64_t)(a.M + 1) * a.K * 2 > ((a.M <= 4 || !pro) ? kSmallMaxBytes : kXldsMaxBytes)) return O355_EUNSUPPORTED;
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

template <typename Kern>
int launch_rot(Kern kern, int gpa, const GemvPlan& p, const GemvArgs& a, hipStream_t stream, const u32x4* w,
               const uint16_t* st, const uint8_t* zt) {
  const size_t lds = (size_t)p.waves * p.nt * 256 * 4 + (size_t)(a.M + 1) * a.K * 2 + (size_t)(a.K >> 7) * (16 / gpa) * 4;
  if (lds > 48 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return O355_ELAUNCH;
  const int ntiles = a.N >> 4;
  const unsigned blocks = p.epi ? (unsigned)(ntiles >> 1) : (unsigned)ntiles;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(p.waves * 64), lds, stream, a, w, st, zt);
  O355_CHECK_LAUNCH();
}

template <typename Kern>
int launch_small(Kern kern, const GemvPlan& p, const GemvArgs& a, hipStream_t stream, const u32x4* w, const uint16_t* st,
                 const uint8_t* zt) {
  const int xbytes = a.M * a.K * 2;
  const int red_off = xbytes + std::max(a.K * 2, 1024);
  const size_t lds = (size_t)red_off + (size_t)p.waves * p.nt * (a.M <= 4 ? 4 : (a.M <= 8 ? 8 : 16)) * 16 * 4;
  if (lds > 48 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return O355_ELAUNCH;
  const int ntiles = a.N >> 4;
  const unsigned blocks = p.epi ? (unsigned)(ntiles >> 1) : (unsigned)((ntiles + p.nt - 1) / p.nt);
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(p.waves * 64), lds, stream, a, w, st, zt);
  O355_CHECK_LAUNCH();
}

#define SMALL_CASE_G(GPAv, NTv, Wv, Pv, Ev)                                                 \
  if (sgpa == GPAv && p.nt == NTv && p.waves == Wv && p.pro == Pv && p.epi == Ev)           \
    return launch_small(w4_gemv_small_kernel<GPAv, NTv, Wv, Pv, Ev>, p, a, as_stream(stream), w, st, zt);
#define SMALL_CASE(NTv, Wv, Pv, Ev) SMALL_CASE_G(4, NTv, Wv, Pv, Ev)
#define SMALL_PLAIN(GPAv)                                                                                        \
  SMALL_CASE_G(GPAv, 1, 4, 0, 0) SMALL_CASE_G(GPAv, 1, 8, 0, 0) SMALL_CASE_G(GPAv, 1, 16, 0, 0)                   \
  SMALL_CASE_G(GPAv, 2, 4, 0, 1) SMALL_CASE_G(GPAv, 2, 8, 0, 1) SMALL_CASE_G(GPAv, 2, 16, 0, 1)
#define SMALL_WAVES(NTv, Pv, Ev) SMALL_CASE(NTv, 4, Pv, Ev) SMALL_CASE(NTv, 8, Pv, Ev) SMALL_CASE(NTv, 16, Pv, Ev)
#define SMALL_FORMS                                                                              \
  SMALL_WAVES(1, 0, 0) SMALL_WAVES(1, 1, 0) SMALL_WAVES(1, 4, 0) SMALL_WAVES(2, 0, 1) \
  SMALL_WAVES(2, 1, 1) SMALL_WAVES(2, 4, 1) SMALL_WAVES(1, 8, 0) SMALL_WAVES(2, 8, 1) \
  SMALL_WAVES(1, 9, 0) SMALL_WAVES(2, 9, 1) SMALL_WAVES(1, 10, 0) SMALL_WAVES(2, 10, 1)

#define ROT_CASE(GPAv, NTv, Wv, Pv, Ev)                                                   \
  if (gpa == GPAv && p.nt == NTv && p.waves == Wv && p.pro == Pv && p.epi == Ev)          \
    return launch_rot(w4_gemv_rot_kernel<GPAv, NTv, Wv, Pv, Ev>, gpa, p, a, as_stream(stream), w, st, zt);
#define ROT_WAVES(GPAv, NTv, Pv, Ev) ROT_CASE(GPAv, NTv, 4, Pv, Ev) ROT_CASE(GPAv, NTv, 8, Pv, Ev) ROT_CASE(GPAv, NTv, 16, Pv, Ev)
#define ROT_FORMS(GPAv)                                                                        \
  ROT_WAVES(GPAv, 1, 0, 0) ROT_WAVES(GPAv, 1, 1, 0) ROT_WAVES(GPAv, 1, 4, 0) ROT_WAVES(GPAv, 2, 0, 1) \
  ROT_WAVES(GPAv, 2, 1, 1) ROT_WAVES(GPAv, 2, 4, 1)

// 5 .. 8 rows through w4_gemv_r8_kernel.  nt / waves 0: chosen here (measured on the 7B shapes at 8 rows: three tiles
// per workgroup where that still leaves a workgroup per CU, two up-and-gate pairs for the SwiGLU form).
template <typename Kern>
int launch_r8(Kern kern, int nt, int waves, bool epi, int n_cu, const GemvArgs& a, hipStream_t stream, const u32x4* w,
              const uint16_t* st, const uint8_t* zt) {
  const size_t lds = (size_t)2 * waves * nt * 128 * 4 + 32 + (size_t)waves * kR8WaveBytes;
  if (lds > 48 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return O355_ELAUNCH;
  const int ntiles = a.N >> 4;
  const int sets = epi ? ((ntiles >> 1) + (nt >> 1) - 1) / (nt >> 1) : (ntiles + nt - 1) / nt;
  hipLaunchKernelGGL(kern, dim3((unsigned)std::min(sets, n_cu)), dim3(waves * 64), lds, stream, a, w, st, zt);
  O355_CHECK_LAUNCH();
}

#define R8_CASE(NTv, Wv, Pv, PROv, Ev, PFv)                                                            \
  if (nt == NTv && waves == Wv && pmax == Pv && pro == PROv && epi == (Ev == 1) && pf == PFv)           \
    return launch_r8(w4_gemv_r8_kernel<NTv, Wv, Pv, PROv, Ev, PFv>, nt, waves, epi, n_cu, a, as_stream(stream), w, st, zt);

// The instantiations that exist: those that fit the register file of their workgroup size without spilling
// (16 waves: 128 registers per lane; 8 waves: 256).  pmax pairs of groups per wave, all requested up front; pf: a
// second set of weight registers.
constexpr bool r8_exists(int nt, int waves, int pmax, bool pro, bool epi, bool pf) {
  if (pmax < 1 || pmax > (pro ? 2 : 3)) return false;
  if (epi ? (nt != 2 && nt != 4) : (nt < 1 || nt > 3)) return false;
  if (waves == 8) {
    if (pf) return nt <= 2 && pmax <= 2;
    return !(nt == 4 && pmax == 3);
  }
  if (waves != 16) return false;
  if (nt == 1 && !epi && pmax <= 2) return true;  // one tile: two pairs fit with the prologue and with the second set
  if (pf) return pmax == 1 && nt <= 2;
  if (pro) return pmax == 1;
  return nt == 1 || pmax == 1;
}

// CUs of the device first used (a grid only has to be about as large as the machine); 0 if the query fails
int cu_count() {
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0)
      n_cu = cus;
  }
  return n_cu;
}

// Up to 8 rows through w4_gemv_rows_kernel when the units of the product can be dealt out over one workgroup per CU
// (at most four tiles or three up/gate pairs each); O355_EUNSUPPORTED otherwise (the caller goes on to the kernel
// that walks sets of tiles).
int w4_rows_dispatch(const GemvArgs& a, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, bool pro, bool epi,
                     void* stream) {
  const int G = a.K >> 7, ntiles = a.N >> 4, n_cu = std::max(cu_count(), 1);
  const int units = epi ? ntiles >> 1 : ntiles;
  // 16 waves from 32 groups on, unless the groups split much more evenly into pairs over 8 (K = 5120: 16 runs of 2 or
  // 3 groups -- two pairs each, a third of them empty -- or 8 runs of 5), as measured for the set-walking kernel
  auto pairs_of = [&](int wv) { return std::max(1, ((G + wv - 1) / wv + 1) >> 1); };
  const double fill16 = (double)G / (2.0 * pairs_of(16) * 16), fill8 = (double)G / (2.0 * pairs_of(8) * 8);
  const int waves = G >= 32 && !(fill8 > fill16 + 0.15) ? 16 : 8;
  if (G < waves) return O355_EUNSUPPORTED;
  const int np = pairs_of(waves);
  const int prov = !pro ? 0 : (a.K <= 4096 ? 1 : (a.K <= 8192 ? 2 : -1));
  const int per = (units + n_cu - 1) / n_cu;
  if (prov < 0 || np > 3 || per > (epi ? 3 : 4)) return O355_EUNSUPPORTED;
  const int nt = epi ? 2 * per : per;
  // registers of the pieces in flight (weights, rows, and with the prologue the residual and the norm weight): past
  // these counts the instantiations spill (128 registers per lane at 16 waves, 256 at 8)
  if (nt * np * 8 + np * 16 + (pro ? np * 20 : 0) > (waves == 16 ? 90 : 208)) return O355_EUNSUPPORTED;
  const size_t lds = (size_t)waves * nt * 128 * 4 + 32 + (size_t)waves * kR8WaveBytes;
  if (lds > 160 * 1024) return O355_EUNSUPPORTED;
  const unsigned blocks = (unsigned)(per == 1 ? units : n_cu);
  const u32x4* w = (const u32x4*)wt;
  hipStream_t s = as_stream(stream);
#define ROWS_CASE(Wv, Pv, Ev, Nv, Uv)                                                                                  \
  if (waves == Wv && prov == Pv && (int)epi == Ev && np == Nv && per == Uv) {                                          \
    auto kern = w4_gemv_rows_kernel<Wv, Pv, Ev, Nv, Uv>;                                                               \
    if (lds > 48 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                               (int)lds) != hipSuccess)                                                \
      return O355_ELAUNCH;                                                                                             \
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(Wv * 64), lds, s, a, w, st, zt, units);                                \
    O355_CHECK_LAUNCH();                                                                                               \
  }
#define ROWS_FORMS(Wv, Pv, Nv)                                                                                    \
  ROWS_CASE(Wv, Pv, 0, Nv, 1) ROWS_CASE(Wv, Pv, 0, Nv, 2) ROWS_CASE(Wv, Pv, 0, Nv, 3) ROWS_CASE(Wv, Pv, 0, Nv, 4) \
  ROWS_CASE(Wv, Pv, 1, Nv, 1) ROWS_CASE(Wv, Pv, 1, Nv, 2) ROWS_CASE(Wv, Pv, 1, Nv, 3)
  ROWS_FORMS(16, 0, 1) ROWS_FORMS(16, 0, 2) ROWS_FORMS(16, 0, 3) ROWS_FORMS(16, 1, 1) ROWS_FORMS(16, 2, 2)
  ROWS_FORMS(8, 0, 1) ROWS_FORMS(8, 0, 3) ROWS_FORMS(8, 1, 1) ROWS_FORMS(8, 2, 3)
#undef ROWS_FORMS
#undef ROWS_CASE
  return O355_EUNSUPPORTED;
}

int w4_r8_dispatch(const GemvArgs& a, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, bool pro, bool epi, int nt,
                   int waves, void* stream) {
  const int G = a.K >> 7, ntiles = a.N >> 4;
  if (a.M < 1 || a.M > 8 || (a.K & 127) || (a.N & 15) || (epi && (a.N & 31))) return O355_EUNSUPPORTED;
  if ((int64_t)a.M * a.K * 2 >= 0x40000000 || (int64_t)ntiles * G * 1024 >= (1ll << 31)) return O355_EUNSUPPORTED;
  if (pro && (!a.ssq_in || !a.resid || !a.norm_w || !a.x_out || (a.K >> 4) > 1024)) return O355_EUNSUPPORTED;
  if (a.ssq_out && epi) return O355_EUNSUPPORTED;
  if (nt == 0 && waves == 0) {  // no form asked for: the kernel that issues everything at once, where it covers the shape
    const int st_rows = w4_rows_dispatch(a, wt, st, zt, pro, epi, stream);
    if (st_rows != O355_EUNSUPPORTED) return st_rows;
  }
  static int n_cu = 0;  // of the device first used: the grid only has to be about as large as the machine
  if (n_cu == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      return O355_ELAUNCH;
    n_cu = cus;
  }
  // a workgroup walks its sets of tiles one after the other: small sets, few registers; two tiles per set once a
  // workgroup would walk more than eight sets (measured at 8 rows, N = 100352: 41.7 against 47.6 us)
  const bool auto_nt = nt == 0;
  if (auto_nt) nt = epi ? 2 : (ntiles > 8 * n_cu ? 2 : 1);
  auto pairs_of = [&](int wv) { return std::max(1, ((G + wv - 1) / wv + 1) >> 1); };  // of the wave with the longest run
  auto sets_of = [&](int t) { return epi ? ((ntiles >> 1) + (t >> 1) - 1) / (t >> 1) : (ntiles + t - 1) / t; };
  auto any16 = [&](int t) { return r8_exists(t, 16, pairs_of(16), pro, epi, sets_of(t) > n_cu) || r8_exists(t, 16, pairs_of(16), pro, epi, false); };
  auto any8 = [&](int t) { return r8_exists(t, 8, pairs_of(8), pro, epi, sets_of(t) > n_cu) || r8_exists(t, 8, pairs_of(8), pro, epi, false); };
  if (waves == 0) {
    // 16 waves where an instantiation exists, unless the groups split much more evenly into pairs over 8 (K = 5120:
    // 40 groups are 16 runs of 2 or 3 -- two pairs each, a third of them empty -- or 8 runs of 5; measured at 8 rows,
    // N = 13824: 14.2 against 12.8 us with two tiles per set)
    const double fill16 = (double)G / (2.0 * pairs_of(16) * 16), fill8 = (double)G / (2.0 * pairs_of(8) * 8);
    const int nt8 = (auto_nt && !epi && nt == 1 && any8(2)) ? 2 : nt;
    if (G >= 32 && any16(nt) && !(fill8 > fill16 + 0.15 && any8(nt8))) {
      waves = 16;
    } else {
      waves = 8;
      nt = nt8;
    }
  }
  const int sets = sets_of(nt);
  const bool want_pf = sets > n_cu;
  const int pmax = pairs_of(waves);
  bool pf = want_pf;
  if (pf && !r8_exists(nt, waves, pmax, pro, epi, true)) pf = false;
  if (!r8_exists(nt, waves, pmax, pro, epi, pf)) return O355_EUNSUPPORTED;
  const u32x4* w = (const u32x4*)wt;
  // 16 waves
  R8_CASE(1, 16, 1, false, 0, false) R8_CASE(1, 16, 2, false, 0, false) R8_CASE(1, 16, 3, false, 0, false) R8_CASE(1, 16, 1, true, 0, false)
  R8_CASE(2, 16, 1, false, 0, false) R8_CASE(2, 16, 1, true, 0, false)
  R8_CASE(3, 16, 1, false, 0, false) R8_CASE(3, 16, 1, true, 0, false)
  R8_CASE(2, 16, 1, false, 1, false) R8_CASE(2, 16, 1, true, 1, false)
  R8_CASE(4, 16, 1, false, 1, false) R8_CASE(4, 16, 1, true, 1, false)
  R8_CASE(1, 16, 2, true, 0, false) R8_CASE(1, 16, 2, true, 0, true) R8_CASE(1, 16, 2, false, 0, true)
  R8_CASE(1, 16, 1, false, 0, true) R8_CASE(1, 16, 1, true, 0, true) R8_CASE(2, 16, 1, false, 0, true) R8_CASE(2, 16, 1, true, 0, true)
  R8_CASE(2, 16, 1, false, 1, true) R8_CASE(2, 16, 1, true, 1, true)
  // 8 waves
  R8_CASE(1, 8, 1, false, 0, false) R8_CASE(1, 8, 2, false, 0, false) R8_CASE(1, 8, 3, false, 0, false) R8_CASE(1, 8, 1, true, 0, false) R8_CASE(1, 8, 2, true, 0, false)
  R8_CASE(2, 8, 1, false, 0, false) R8_CASE(2, 8, 2, false, 0, false) R8_CASE(2, 8, 3, false, 0, false) R8_CASE(2, 8, 1, true, 0, false) R8_CASE(2, 8, 2, true, 0, false)
  R8_CASE(3, 8, 1, false, 0, false) R8_CASE(3, 8, 2, false, 0, false) R8_CASE(3, 8, 3, false, 0, false) R8_CASE(3, 8, 1, true, 0, false) R8_CASE(3, 8, 2, true, 0, false)
  R8_CASE(2, 8, 1, false, 1, false) R8_CASE(2, 8, 2, false, 1, false) R8_CASE(2, 8, 3, false, 1, false) R8_CASE(2, 8, 1, true, 1, false) R8_CASE(2, 8, 2, true, 1, false)
  R8_CASE(4, 8, 1, false, 1, false) R8_CASE(4, 8, 2, false, 1, false) R8_CASE(4, 8, 1, true, 1, false) R8_CASE(4, 8, 2, true, 1, false)
  R8_CASE(1, 8, 1, false, 0, true) R8_CASE(1, 8, 2, false, 0, true) R8_CASE(1, 8, 1, true, 0, true) R8_CASE(1, 8, 2, true, 0, true)
  R8_CASE(2, 8, 1, false, 0, true) R8_CASE(2, 8, 2, false, 0, true) R8_CASE(2, 8, 1, true, 0, true) R8_CASE(2, 8, 2, true, 0, true)
  R8_CASE(2, 8, 1, false, 1, true) R8_CASE(2, 8, 2, false, 1, true) R8_CASE(2, 8, 1, true, 1, true) R8_CASE(2, 8, 2, true, 1, true)
  return O355_EUNSUPPORTED;
}

// One row through w4_gemv_one_kernel; O355_EUNSUPPORTED for what it does not cover (the caller goes on to the
// general kernels).  `pro`: chained norm prologue (ssq_in given).
int w4_one_dispatch(const GemvArgs& a, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, bool pro, bool epi,
                    void* stream) {
  const int G = a.K >> 7, ntiles = a.N >> 4;
  if (a.M != 1 || (a.K & 127) || a.K < 512 || (a.N & 15) || (epi && (a.N & 31)) || (pro && !a.ssq_in) || (epi && a.ssq_out))
    return O355_EUNSUPPORTED;
  if ((int64_t)ntiles * G * 1024 >= (1ll << 31)) return O355_EUNSUPPORTED;  // 32-bit offsets into the weights
  const int waves = (epi ? ntiles >> 1 : ntiles) <= 512 && G >= 16 ? 16 : 8;  // as measured for the kernel above: narrow outputs take 16
  if (G < waves) return O355_EUNSUPPORTED;
  const int ngv = (G + waves - 1) / waves;  // groups of the longest run; the others have one less or as many
  const int prov = !pro ? 0 : (a.K <= 4096 ? 1 : (a.K <= 8192 ? 2 : -1));
  if (ngv > 8 || prov < 0) return O355_EUNSUPPORTED;
  // tiles (pairs) per workgroup: the count that leaves the busiest CU the fewest tiles when the workgroups are dealt
  // out evenly, the larger on ties (7B att_proj: 768 tiles = 256 workgroups of three)
  const int units = epi ? ntiles >> 1 : ntiles, n_cu = std::max(cu_count(), 1);
  int per = 1;
  if (!epi && waves == 8 && ngv <= 4 && units % 3 == 0 && ((units / 3 + n_cu - 1) / n_cu) * 3 <= (units + n_cu - 1) / n_cu) per = 3;
  const int nt = epi ? 2 * per : per;
  const size_t lds = (size_t)a.K * 4 + (size_t)waves * nt * 64;
  if (lds > 160 * 1024) return O355_EUNSUPPORTED;
  OneArgs o{a.x, a.resid, a.norm_w, a.x_out, a.ssq_in, (const u32x4*)wt, st, zt, a.y, a.ssq_out, a.eps, (float)a.K, a.K, G,
            ntiles >> 1, (uint32_t)((int64_t)ntiles * G * 1024), (uint32_t)((int64_t)ntiles * G * 32), (uint32_t)((int64_t)ntiles * G * 8)};
  const unsigned blocks = (unsigned)(units / per);
  hipStream_t s = as_stream(stream);
#define ONE_CASE(Wv, Pv, Ev, Gv, Nv)                                                                                   \
  if (waves == Wv && prov == Pv && (int)epi == Ev && ngv == Gv && nt == Nv) {                                          \
    auto kern = w4_gemv_one_kernel<Wv, Pv, Ev, Gv, Nv>;                                                                \
    if (lds > 48 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                               (int)lds) != hipSuccess)                                                \
      return O355_ELAUNCH;                                                                                             \
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(Wv * 64), lds, s, o);                                                  \
    O355_CHECK_LAUNCH();                                                                                               \
  }
  // per (waves, groups): plain and SwiGLU, each without and with the prologue that the K of that split can have
  // (K <= 4096: one request for the sums of squares, K <= 8192: two); three tiles per workgroup for 8 waves of <= 4 groups
#define ONE_PAIR(Wv, Pv, Gv) ONE_CASE(Wv, Pv, 0, Gv, 1) ONE_CASE(Wv, Pv, 1, Gv, 2)
#define ONE_W8_LOW(Gv) ONE_PAIR(8, 0, Gv) ONE_PAIR(8, 1, Gv) ONE_CASE(8, 0, 0, Gv, 3) ONE_CASE(8, 1, 0, Gv, 3)
#define ONE_W8_HIGH(Gv) ONE_PAIR(8, 0, Gv) ONE_PAIR(8, 2, Gv)
  ONE_W8_LOW(1) ONE_W8_LOW(2) ONE_W8_LOW(3) ONE_W8_LOW(4) ONE_W8_HIGH(5) ONE_W8_HIGH(6) ONE_W8_HIGH(7) ONE_W8_HIGH(8)
  ONE_PAIR(16, 0, 1) ONE_PAIR(16, 1, 1) ONE_PAIR(16, 0, 2) ONE_PAIR(16, 1, 2) ONE_PAIR(16, 0, 3) ONE_PAIR(16, 2, 3)
  ONE_PAIR(16, 0, 4) ONE_PAIR(16, 2, 4) ONE_PAIR(16, 0, 5) ONE_PAIR(16, 0, 6) ONE_PAIR(16, 0, 7) ONE_PAIR(16, 0, 8)
#undef ONE_W8_HIGH
#undef ONE_W8_LOW
#undef ONE_PAIR
#undef ONE_CASE
  return O355_EUNSUPPORTED;
}

int w4_gemv_dispatch(const GemvArgs& a, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, bool pro, bool epi,
                     void* stream, int form = kFormChoose) {
  if (a.M == 1 && form == kFormChoose && (!pro || a.ssq_in)) {  // one row: the kernel written for it
    const int st1 = w4_one_dispatch(a, wt, st, zt, pro, epi, stream);
    if (st1 != O355_EUNSUPPORTED) return st1;
  }
  GemvPlan p = plan_gemv(a.M, a.N, a.K, true, pro, epi);
  const u32x4* w = (const u32x4*)wt;
  const int sgpa = a.M <= 4 ? 4 : (a.M <= 8 ? 2 : 1);
  const bool small_ok = a.M <= 16 && (a.M <= 4 || p.pro == 0) && (int64_t)(a.M + 1) * a.K * 2 <= kSmallMaxBytes && (int64_t)(a.N >> 4) * (a.K >> 7) * 1024 < (1ll << 31) && form != kFormOlder;
  // Plain products with many columns: from 9 rows (8 for wide outputs; measured at N = 12288, K = 4096: 5 rows 8.7
  // against 11.3 us, 8 rows 11.2 against 10.8) the staged-activation kernel
  // wins over the kernels below, which keep all rows of x in LDS per workgroup (measured).
  const bool plain = !pro && !epi && !a.ssq_in && !a.ssq_out;
  const bool mid_wins = a.M > 16 || (a.M > 8 && a.N >= 8192) || (a.M > 7 && a.N >= 12288);
  const bool force_mid = form == kFormMid || form == kFormMid1 || form == kFormMid2;
  if (plain && a.M > 4 && a.M <= 8 && form == kFormChoose) {  // measured at 8 rows: 8.7 / 4.8 / 8.6 us against 11.0 / 4.9 / 10.6
    const int st8 = w4_r8_dispatch(a, wt, st, zt, false, false, 0, 0, stream);
    if (st8 != O355_EUNSUPPORTED) return st8;
  }
  if (plain && ((mid_wins && form == kFormChoose) || force_mid)) {
    const int pairs = form == kFormMid1 ? 1 : (form == kFormMid2 ? 2 : 0);
    const int st_mid = o355_w4_mid_dispatch(a.x, wt, st, zt, a.y, a.M, a.N, a.K, pairs, stream);
    if (st_mid != O355_EUNSUPPORTED || force_mid) return st_mid;  // else: sizes beyond its 32-bit offsets
  }
  if ((a.ssq_in || a.ssq_out) && a.M > 4) return w4_r8_dispatch(a, wt, st, zt, pro, epi, 0, 0, stream);
  if (a.ssq_in && a.M > 1) {
    // two to four rows with the chained prologue: the kernel below needs two or four pieces of x per lane for them
    // and with those registers one or two of its workgroups fit a CU (measured, att_proj / ff_proj: 2 rows 16.4 /
    // 21.7 against 8.9 / 12.6 us, 4 rows 37 / 64 against 9.6 / 13.2)
    const int st8 = w4_r8_dispatch(a, wt, st, zt, pro, epi, 0, 0, stream);
    if (st8 != O355_EUNSUPPORTED) return st8;
  }
  if (a.ssq_in || a.ssq_out) {  // chained norms: only the lean kernels speak that protocol
    if (!small_ok || a.M > 4 || (a.ssq_out && epi)) return O355_EUNSUPPORTED;
    if (a.ssq_in) {
      const int slice_kib = ((((a.K >> 7) + p.waves - 1) / p.waves) * 256 + 1023) >> 10;  // per row, largest wave
      const int pieces = a.M * slice_kib;
      if (!pro || pieces > kChainPieces || (a.K >> 4) > 1024) return O355_EUNSUPPORTED;
      p.pro = pieces <= 1 ? 8 : (pieces <= 2 ? 9 : 10);
    }
  }
  if (small_ok && p.pro >= 0) {
    SMALL_FORMS
    SMALL_PLAIN(2)
    SMALL_PLAIN(1)
    return O355_EUNSUPPORTED;
  }
  if (p.mt == 1 && p.xlds) {  // M <= 16 with the activations in LDS: accumulators shared between groups
    const int gpa = a.M <= 4 ? 4 : (a.M <= 8 ? 2 : 1);
    ROT_FORMS(4)
    ROT_FORMS(2)
    ROT_FORMS(1)
    return O355_EUNSUPPORTED;
  }
  GEMV_WAVES(w4_gemv_kernel, 1, 1, 2, false, 0, 0, w, st, zt)
  GEMV_WAVES(w4_gemv_kernel, 2, 1, 2, false, 0, 0, w, st, zt)
  GEMV_WAVES(w4_gemv_kernel, 4, 1, 2, false, 0, 0, w, st, zt)
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

extern "C" int olmo355_w4_gemv_form(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                                    uint16_t* y, int M, int N, int K, int form, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0 || form < kFormChoose || form > kFormOlder) return O355_EINVAL;
  if (M > 64 || (K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  const GemvArgs a{x, nullptr, nullptr, nullptr, y, 0.f, M, N, K};
  return w4_gemv_dispatch(a, wt, st, zt, false, false, stream, form);
}

extern "C" int olmo355_w4_gemv(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                               uint16_t* y, int M, int N, int K, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (M > 64 || (K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  const GemvArgs a{x, nullptr, nullptr, nullptr, y, 0.f, M, N, K};
  return w4_gemv_dispatch(a, wt, st, zt, false, false, stream);
}

// fp16 activations in, fp16 out (QuantLinear.forward on fp16 input, qlinear_cuda_old.py:287-290), up to 16 rows that fit
// LDS with a zero row; O355_EUNSUPPORTED otherwise (olmo355_w4_gemm_f16 takes any M).
extern "C" int olmo355_w4_gemv_f16(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                                   uint16_t* y, int M, int N, int K, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (M > 16 || (K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  if ((int64_t)(M + 1) * K * 2 > kSmallMaxBytes || (int64_t)(N >> 4) * (K >> 7) * 1024 >= (1ll << 31)) return O355_EUNSUPPORTED;
  const GemvArgs a{x, nullptr, nullptr, nullptr, y, 0.f, M, N, K};
  const GemvPlan p = plan_gemv(M, N, K, true, false, false);
  const u32x4* w = (const u32x4*)wt;
  const int sgpa = M <= 4 ? 4 : (M <= 8 ? 2 : 1);
#define SMALL_F16(GPAv, Wv)                          \
  if (sgpa == GPAv && p.waves == Wv)                 \
    return launch_small(w4_gemv_small_kernel<GPAv, 1, Wv, 0, 0, true>, p, a, as_stream(stream), w, st, zt);
  SMALL_F16(4, 4) SMALL_F16(4, 8) SMALL_F16(4, 16) SMALL_F16(2, 4) SMALL_F16(2, 8) SMALL_F16(2, 16) SMALL_F16(1, 4) SMALL_F16(1, 8)
  SMALL_F16(1, 16)
#undef SMALL_F16
  return O355_EUNSUPPORTED;
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

extern "C" int olmo355_w4_gemv_chain(const uint16_t* x, const uint16_t* resid, const uint16_t* norm_w, float eps,
                                     uint16_t* x_out, const float* ssq_in, const uint32_t* wt, const uint16_t* st,
                                     const uint8_t* zt, uint16_t* y, float* ssq_out, int M, int N, int K, int swiglu,
                                     void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if ((resid != nullptr) != (ssq_in != nullptr)) return O355_EINVAL;  // the prologue here is the chained one
  if (M > 8 || (K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  GemvArgs a{x, resid, norm_w, x_out, y, eps, M, N, K};
  a.ssq_in = ssq_in, a.ssq_out = ssq_out;
  const bool pro = resid != nullptr, epi = swiglu != 0;
  if (M > 4) return w4_r8_dispatch(a, wt, st, zt, pro, epi, 0, 0, stream);
  const int chk = check_fused(a, pro, epi);
  if (chk != O355_OK) return chk;
  return w4_gemv_dispatch(a, wt, st, zt, pro, epi, stream);
}

extern "C" int olmo355_w4_gemv_r8_form(const uint16_t* x, const uint16_t* resid, const uint16_t* norm_w, float eps,
                                       uint16_t* x_out, const float* ssq_in, const uint32_t* wt, const uint16_t* st,
                                       const uint8_t* zt, uint16_t* y, float* ssq_out, int M, int N, int K, int swiglu,
                                       int nt, int waves, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0 || nt < 0 || (waves != 0 && waves != 8 && waves != 16))
    return O355_EINVAL;
  if ((resid != nullptr) != (ssq_in != nullptr)) return O355_EINVAL;
  GemvArgs a{x, resid, norm_w, x_out, y, eps, M, N, K};
  a.ssq_in = ssq_in, a.ssq_out = ssq_out;
  return w4_r8_dispatch(a, wt, st, zt, resid != nullptr, swiglu != 0, nt, waves, stream);
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
