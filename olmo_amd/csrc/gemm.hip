// Large-M linear layers (prefill): y[M,N] = x[M,K] . W[K,N] on the matrix cores
// (v_mfma_f32_16x16x32_bf16), fp32 accumulation, bf16 output.
//
// Workgroup = 4 waves in a 2x2 arrangement over a BM x BN output tile, K advanced 64 at a
// time.  Both operands are staged in LDS in *fragment-major* order -- [16-row tile][k-step of
// 32][64 lanes][16 bytes] -- so every MFMA operand is one conflict-free ds_read_b128, and
// each 16-byte global load lands in exactly one LDS slot.  LDS is double-buffered: while the
// matrix cores work on stage s the same waves write stage s+1 (for int4 weights: unpack the
// tiled words, apply scale and zero in fp32, round to bf16) and fetch stage s+2 from memory
// into registers; one barrier per stage.
//
// The int4 operand is W = bf16(scale * (q - zero)) (fp32 product, one rounding).
#include "common.h"

namespace {

constexpr int BK = 64;

__device__ __forceinline__ int xcd_swizzle(int pid, int nblocks) {
  // consecutive workgroup ids go round-robin over the 8 XCDs; give each XCD a contiguous
  // range of tiles so that tiles sharing a weight panel share an L2
  const int per = nblocks / 8;
  if (per * 8 != nblocks) return pid;
  return (pid % 8) * per + pid / 8;
}

// dequantise one tiled word (8 weights of one column) to 8 bf16 in MFMA operand order
__device__ __forceinline__ u32x4 dequant_word_bf16(uint32_t w, float s, float c) {
  // c = -(128 + zero) * s ; value = (128+q)*s + c = s*(q - zero), single fp32 rounding of the fma
  u32x4 o;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const uint32_t p = ((w >> (4 * t)) & 0x000f000fu) | 0x43004300u;
    const float lo = __builtin_fmaf(bf16lo_to_f32(p), s, c);
    const float hi = __builtin_fmaf(bf16hi_to_f32(p), s, c);
    o[t] = pack_bf16x2(lo, hi);
  }
  return o;
}

template <int WMT, int WNT, bool W4>
__global__ __launch_bounds__(256) void gemm_kernel(const uint16_t* __restrict__ x, const uint32_t* __restrict__ wt,
                                                   const uint16_t* __restrict__ st, const uint8_t* __restrict__ zt,
                                                   uint16_t* __restrict__ y, int M, int N, int K, int tiles_m,
                                                   int tiles_n) {
  constexpr int BM = 32 * WMT, BN = 32 * WNT;
  constexpr int A_FRAGS = (BM / 16) * 2, B_FRAGS = (BN / 16) * 2;  // per stage: tiles x 2 k-steps
  constexpr int A_LD = (BM * 8) / 256;                               // 16-byte chunks per thread per stage
  constexpr int B_ITEMS = (BN / 16) * 64 / 256;                      // (n-tile, lane) items per thread per stage
  extern __shared__ __align__(16) unsigned char smem[];
  u32x4* lds_a = reinterpret_cast<u32x4*>(smem);                     // [2][A_FRAGS][64]
  u32x4* lds_b = lds_a + 2 * A_FRAGS * 64;                           // [2][B_FRAGS][64]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int pid = xcd_swizzle(blockIdx.x, tiles_m * tiles_n);
  const int tile_m = pid % tiles_m, tile_n = pid / tiles_m;
  const int m0 = tile_m * BM, nt0 = tile_n * (BN / 16);
  const int ntiles = N >> 4;
  const int G = K >> 7, KS = K >> 5;
  const int stages = K / BK;

  // ---- global -> register staging -----------------------------------------------------------
  u32x4 ra[A_LD];
  u32x2 rbw[B_ITEMS];  // int4: two tiled words (k-steps 2h, 2h+1)
  u32x4 rbd[W4 ? 1 : B_ITEMS][2];
  float rs[B_ITEMS], rc[B_ITEMS];

  auto fetch = [&](int s) {
    const int k0 = s * BK;
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
      const int row = (tid >> 3) + 32 * i, c = tid & 7;
      const int gm = m0 + row;
      if (gm < M) ra[i] = *reinterpret_cast<const u32x4*>(x + (int64_t)gm * K + k0 + 8 * c);
      else ra[i] = u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int i = 0; i < B_ITEMS; ++i) {
      const int nt = min(nt0 + (tid >> 6) + 4 * i, ntiles - 1);
      if constexpr (W4) {
        const int g = k0 >> 7, h = (k0 >> 6) & 1;
        const int64_t tile = (int64_t)nt * G + g;
        rbw[i] = *reinterpret_cast<const u32x2*>(wt + (tile * 64 + lane) * 4 + 2 * h);
        const int col = lane & 15;
        const float sc = (float)__builtin_bit_cast(_Float16, st[tile * 16 + col]);
        const int z = 129 + (int)((zt[tile * 8 + (col >> 1)] >> (4 * (col & 1))) & 15u);
        rs[i] = sc;
        rc[i] = -(float)z * sc;
      } else {
        const u32x4* src = reinterpret_cast<const u32x4*>(wt) + ((int64_t)nt * KS + (k0 >> 5)) * 64 + lane;
        rbd[i][0] = src[0];
        rbd[i][1] = src[64];
      }
    }
  };

  auto stash = [&](int buf) {
    u32x4* a = lds_a + buf * A_FRAGS * 64;
    u32x4* b = lds_b + buf * B_FRAGS * 64;
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
      const int row = (tid >> 3) + 32 * i, c = tid & 7;
      a[((row >> 4) * 2 + (c >> 2)) * 64 + (row & 15) + 16 * (c & 3)] = ra[i];
    }
#pragma unroll
    for (int i = 0; i < B_ITEMS; ++i) {
      const int ntl = (tid >> 6) + 4 * i;
      if constexpr (W4) {
        b[(ntl * 2 + 0) * 64 + lane] = dequant_word_bf16(rbw[i].x, rs[i], rc[i]);
        b[(ntl * 2 + 1) * 64 + lane] = dequant_word_bf16(rbw[i].y, rs[i], rc[i]);
      } else {
        b[(ntl * 2 + 0) * 64 + lane] = rbd[i][0];
        b[(ntl * 2 + 1) * 64 + lane] = rbd[i][1];
      }
    }
  };

  f32x4 acc[WMT][WNT];
#pragma unroll
  for (int i = 0; i < WMT; ++i)
#pragma unroll
    for (int j = 0; j < WNT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  fetch(0);
  stash(0);
  if (stages > 1) fetch(1);
  __syncthreads();

  for (int s = 0; s < stages; ++s) {
    const int buf = s & 1;
    const u32x4* a = lds_a + buf * A_FRAGS * 64;
    const u32x4* b = lds_b + buf * B_FRAGS * 64;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      bf16x8 af[WMT], bfr[WNT];
#pragma unroll
      for (int i = 0; i < WMT; ++i) af[i] = __builtin_bit_cast(bf16x8, a[((wm * WMT + i) * 2 + ks) * 64 + lane]);
#pragma unroll
      for (int j = 0; j < WNT; ++j) bfr[j] = __builtin_bit_cast(bf16x8, b[((wn * WNT + j) * 2 + ks) * 64 + lane]);
#pragma unroll
      for (int i = 0; i < WMT; ++i)
#pragma unroll
        for (int j = 0; j < WNT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    if (s + 1 < stages) stash(buf ^ 1);
    if (s + 2 < stages) fetch(s + 2);
    __syncthreads();
  }

  // ---- epilogue: D[m = 4*(lane>>4)+r][n = lane&15] ---------------------------------------------
#pragma unroll
  for (int i = 0; i < WMT; ++i)
#pragma unroll
    for (int j = 0; j < WNT; ++j) {
      const int nt = nt0 + wn * WNT + j;
      if (nt >= ntiles) continue;
      const int n = nt * 16 + (lane & 15);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m0 + (wm * WMT + i) * 16 + 4 * (lane >> 4) + r;
        if (m < M) y[(int64_t)m * N + n] = f32_to_bf16_bits(acc[i][j][r]);
      }
    }
}

template <int WMT, int WNT, bool W4>
int launch_gemm(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y, int M, int N,
                int K, hipStream_t stream) {
  constexpr int BM = 32 * WMT, BN = 32 * WNT;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const size_t lds = (size_t)2 * ((BM / 16) * 2 + (BN / 16) * 2) * 64 * 16;
  auto kern = gemm_kernel<WMT, WNT, W4>;
  if (lds > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) !=
        hipSuccess)
      return O355_ELAUNCH;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n)), dim3(256), lds, stream, x, wt, st, zt, y, M, N, K,
                     tiles_m, tiles_n);
  O355_CHECK_LAUNCH();
}

template <bool W4>
int dispatch_gemm(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y, int M,
                  int N, int K, hipStream_t stream) {
  // Big tiles when they still give at least one workgroup per CU; otherwise smaller ones.
  const int64_t big = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
  if (big >= 256) return launch_gemm<8, 8, W4>(x, wt, st, zt, y, M, N, K, stream);
  const int64_t mid = (int64_t)((M + 255) / 256) * ((N + 127) / 128);
  if (mid >= 256) return launch_gemm<8, 4, W4>(x, wt, st, zt, y, M, N, K, stream);
  return launch_gemm<4, 4, W4>(x, wt, st, zt, y, M, N, K, stream);
}

}  // namespace

extern "C" int olmo355_w4_gemm(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                               uint16_t* y, int M, int N, int K, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if ((K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  return dispatch_gemm<true>(x, wt, st, zt, y, M, N, K, as_stream(stream));
}

extern "C" int olmo355_b16_gemm(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K,
                                void* stream) {
  if (!x || !wt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if ((K & 63) || (N & 15)) return O355_EUNSUPPORTED;
  return dispatch_gemm<false>(x, reinterpret_cast<const uint32_t*>(wt), nullptr, nullptr, y, M, N, K,
                              as_stream(stream));
}

// ---- dense bf16 weight re-tiling: [N,K] row-major -> [N/16][K/32][64 lanes][8] -----------------
namespace {
__global__ __launch_bounds__(256) void b16_repack_kernel(const u32x4* __restrict__ w, u32x4* __restrict__ wt, int N,
                                                         int K) {
  const int KS = K >> 5;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // one 16-byte fragment piece
  const int64_t total = (int64_t)(N >> 4) * KS * 64;
  if (idx >= total) return;
  const int lane = (int)(idx & 63);
  const int64_t t = idx >> 6;
  const int ks = (int)(t % KS), nt = (int)(t / KS);
  const int n = 16 * nt + (lane & 15), k = 32 * ks + 8 * (lane >> 4);
  wt[idx] = w[((int64_t)n * K + k) >> 3];
}

// fp32 reference-precision linear for the fp32 model configuration: y = x . w^T with fp32 FMAs,
// 64x64 tile per workgroup, 4x4 outputs per thread, K staged 16 at a time through LDS.
__global__ __launch_bounds__(256) void f32_linear_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                         float* __restrict__ y, int M, int N, int K) {
  __shared__ float sx[16][64 + 1], sw[16][64 + 1];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += 16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + 256 * i;  // 0..1023 : row (0..63), k (0..15)
      const int r = e >> 4, kk = e & 15;
      const int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
      sx[kk][r] = (gm < M && gk < K) ? x[(int64_t)gm * K + gk] : 0.f;
      sw[kk][r] = (gn < N && gk < K) ? w[(int64_t)gn * K + gk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = sx[kk][ty * 4 + i], b[i] = sw[kk][tx * 4 + i];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m < M && n < N) y[(int64_t)m * N + n] = acc[i][j];
    }
}
}  // namespace

extern "C" int olmo355_b16_repack(const uint16_t* w_nk, uint16_t* wt, int N, int K, void* stream) {
  if (!w_nk || !wt || N <= 0 || K <= 0) return O355_EINVAL;
  if ((K & 31) || (N & 15)) return O355_EUNSUPPORTED;
  const int64_t total = (int64_t)(N >> 4) * (K >> 5) * 64;
  hipLaunchKernelGGL(b16_repack_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, as_stream(stream),
                     (const u32x4*)w_nk, (u32x4*)wt, N, K);
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_f32_linear(const float* x, const float* w_nk, float* y, int M, int N, int K, void* stream) {
  if (!x || !w_nk || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  hipLaunchKernelGGL(f32_linear_kernel, dim3((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64)), dim3(256), 0,
                     as_stream(stream), x, w_nk, y, M, N, K);
  O355_CHECK_LAUNCH();
}
