// Large-M linear layers (prefill): y[M,N] = x[M,K] . W[K,N] on the matrix cores
// (v_mfma_f32_32x32x16_bf16), fp32 accumulation, bf16 output.
//
// Workgroup = 4 waves in a 2x2 arrangement over a BM x BN output tile (up to 256 x 256, one wave
// per SIMD: a single wave sustains the 8-pass 32x32x16 MFMA back to back, which it does not for
// the 4-pass 16x16x32), K advanced 64 at a time.  Both operands are staged in LDS in
// *fragment-major* order -- [32-row tile][k-step of 16][64 lanes][16 bytes] -- so every MFMA operand
// is one conflict-free ds_read_b128 and each 16-byte piece fetched from memory lands in exactly one
// LDS slot.  The activation pieces are written with an XOR swizzle of the slot (the 16 lanes of one
// LDS write cycle hold 2 rows x 8 column chunks, which would otherwise share two bank groups).
// LDS is double-buffered: while the matrix cores work on stage s the same waves write stage s+1
// (for int4 weights: unpack the tiled words, apply scale and zero in fp32, round to bf16) and fetch
// stage s+2 from memory into registers; the staging work is spread between the k-steps of the MFMA
// loop so that the VALU / LDS / memory instructions issue in the shadow of the matrix pipeline; one
// barrier per stage.
//
// The int4 operand is W = bf16(scale * (q - zero)) (fp32 product, one rounding).
#include "common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BK = 64;      // K per stage
constexpr int KSTEPS = 4;   // MFMA k-steps of 16 per stage

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

// Tile order: consecutive workgroup ids go round-robin over the 8 XCDs.  XCD x works on the row
// tiles tile_m == x (mod 8) and walks the column tiles, so the activation panel of a row tile
// (BM x K, the larger operand) stays in that XCD's L2 while the packed weights stream through.
__device__ __forceinline__ void tile_of(int pid, int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
  if ((tiles_m & 7) == 0) {
    const int xcd = pid & 7, local = pid >> 3;
    tile_n = local % tiles_n;
    tile_m = xcd + 8 * (local / tiles_n);
  } else {
    tile_m = pid % tiles_m;
    tile_n = pid / tiles_m;
  }
}

template <int WMT, int WNT, bool W4>  // 32x32 MFMA tiles per wave along M and N
__global__ __launch_bounds__(256) void gemm_kernel(const uint16_t* __restrict__ x, const uint32_t* __restrict__ wt,
                                                   const uint16_t* __restrict__ st, const uint8_t* __restrict__ zt,
                                                   uint16_t* __restrict__ y, int M, int N, int K, int tiles_m,
                                                   int tiles_n) {
  constexpr int BM = 64 * WMT, BN = 64 * WNT;
  constexpr int A_FRAGS = (BM / 32) * KSTEPS, B_FRAGS = (BN / 32) * KSTEPS;  // 1 KiB fragments per stage
  constexpr int A_LD = (BM * 8) / 256;           // 16-byte activation pieces per thread per stage
  constexpr int B_ITEMS = (BN / 16) * 64 / 256;  // (16-column weight tile, lane) items per thread per stage
  extern __shared__ __align__(16) unsigned char smem[];
  u32x4* lds_a = reinterpret_cast<u32x4*>(smem);  // [2][A_FRAGS][64]
  u32x4* lds_b = lds_a + 2 * A_FRAGS * 64;        // [2][B_FRAGS][64]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  int tile_m, tile_n;
  tile_of(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, nt0 = tile_n * (BN / 16);
  const int ntiles = N >> 4;
  const int G = K >> 7, KS = K >> 5;
  const int stages = K / BK;

  // ---- global -> register staging -----------------------------------------------------------
  u32x4 ra[A_LD];
  u32x2 rbw[B_ITEMS];  // int4: two tiled words (32-row steps 2h, 2h+1 of the group)
  u32x4 rbd[W4 ? 1 : B_ITEMS][2];
  float rs[B_ITEMS], rc[B_ITEMS];

  // rows past M are clamped to the last row (their products are computed and never stored): the
  // loop body stays free of branches, which is what lets the compiler interleave it
  auto fetch_a = [&](int s, int i) {
    const int row = (tid >> 3) + 32 * i, c = tid & 7;
    const int gm = min(m0 + row, M - 1);
    ra[i] = *reinterpret_cast<const u32x4*>(x + (int64_t)gm * K + s * BK + 8 * c);
  };
  auto fetch_b = [&](int s, int i) {
    const int k0 = s * BK;
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
  };
  // piece (row, chunk c of 8 columns) -> fragment (row/32, c/2), slot (c&1)*32 + (row%32 ^ 2c mod 16)
  auto stash_a = [&](u32x4* a, int i) {
    const int row = (tid >> 3) + 32 * i, c = tid & 7;
    a[((row >> 5) * KSTEPS + (c >> 1)) * 64 + (c & 1) * 32 + ((row & 31) ^ ((2 * c) & 15))] = ra[i];
  };
  // weight piece of lane l (column l&15 of its 16-column tile, rows 8*(l>>4).. of 32-row step j):
  // fragment (tile/2, 2j + (l>>5)), slot ((l>>4)&1)*32 + (tile&1)*16 + (l&15)
  auto stash_b = [&](u32x4* b, int i) {
    const int ntl = (tid >> 6) + 4 * i;
    const int kq = lane >> 4;
    const int slot = (kq & 1) * 32 + (ntl & 1) * 16 + (lane & 15);
    const int f0 = (ntl >> 1) * KSTEPS + (kq >> 1);
    if constexpr (W4) {
      b[(f0 + 0) * 64 + slot] = dequant_word_bf16(rbw[i].x, rs[i], rc[i]);
      b[(f0 + 2) * 64 + slot] = dequant_word_bf16(rbw[i].y, rs[i], rc[i]);
    } else {
      b[(f0 + 0) * 64 + slot] = rbd[i][0];
      b[(f0 + 2) * 64 + slot] = rbd[i][1];
    }
  };

  f32x16 acc[WMT][WNT];
#pragma unroll
  for (int i = 0; i < WMT; ++i)
#pragma unroll
    for (int j = 0; j < WNT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

#pragma unroll
  for (int i = 0; i < A_LD; ++i) fetch_a(0, i);
#pragma unroll
  for (int i = 0; i < B_ITEMS; ++i) fetch_b(0, i);
#pragma unroll
  for (int i = 0; i < A_LD; ++i) stash_a(lds_a, i);
#pragma unroll
  for (int i = 0; i < B_ITEMS; ++i) stash_b(lds_b, i);
#pragma unroll
  for (int i = 0; i < A_LD; ++i) fetch_a(min(1, stages - 1), i);
#pragma unroll
  for (int i = 0; i < B_ITEMS; ++i) fetch_b(min(1, stages - 1), i);
  lds_barrier();

  const int row32 = lane & 31, kh = lane >> 5;
  for (int s = 0; s < stages; ++s) {
    const int buf = s & 1;
    const u32x4* a = lds_a + buf * A_FRAGS * 64;
    const u32x4* b = lds_b + buf * B_FRAGS * 64;
    u32x4* an = lds_a + (buf ^ 1) * A_FRAGS * 64;
    u32x4* bn = lds_b + (buf ^ 1) * B_FRAGS * 64;
    // the last stage stashes into a buffer nobody reads again and the last two re-fetch the final
    // stage: redundant, but unconditional
    const int sf = min(s + 2, stages - 1);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      bf16x8 af[WMT], bfr[WNT];
      const int aslot = kh * 32 + (row32 ^ ((2 * (2 * ks + kh)) & 15));
#pragma unroll
      for (int i = 0; i < WMT; ++i) af[i] = __builtin_bit_cast(bf16x8, a[((wm * WMT + i) * KSTEPS + ks) * 64 + aslot]);
#pragma unroll
      for (int j = 0; j < WNT; ++j) bfr[j] = __builtin_bit_cast(bf16x8, b[((wn * WNT + j) * KSTEPS + ks) * 64 + lane]);
#pragma unroll
      for (int i = 0; i < WMT; ++i)
#pragma unroll
        for (int j = 0; j < WNT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
      // a quarter of the staging work per k-step, issued behind this step's MFMAs
#pragma unroll
      for (int i = ks; i < A_LD; i += KSTEPS) stash_a(an, i);
#pragma unroll
      for (int i = ks; i < B_ITEMS; i += KSTEPS) stash_b(bn, i);
#pragma unroll
      for (int i = ks; i < A_LD; i += KSTEPS) fetch_a(sf, i);
#pragma unroll
      for (int i = ks; i < B_ITEMS; i += KSTEPS) fetch_b(sf, i);
    }
    lds_barrier();  // orders LDS only: the global loads of stage s+2 stay in flight across it
  }

  // ---- epilogue: D[m = 8*(r/4) + 4*(lane>>5) + r%4][n = lane&31] of each 32x32 tile ---------------------
#pragma unroll
  for (int i = 0; i < WMT; ++i)
#pragma unroll
    for (int j = 0; j < WNT; ++j) {
      const int n = (nt0 >> 1) * 32 + (wn * WNT + j) * 32 + (lane & 31);
      if (n >= N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + (wm * WMT + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (m < M) y[(int64_t)m * N + n] = f32_to_bf16_bits(acc[i][j][r]);
      }
    }
}

template <int WMT, int WNT, bool W4>
int launch_gemm(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y, int M, int N,
                int K, hipStream_t stream) {
  constexpr int BM = 64 * WMT, BN = 64 * WNT;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const size_t lds = (size_t)2 * ((BM / 32) + (BN / 32)) * KSTEPS * 64 * 16;
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
  if (big >= 256) return launch_gemm<4, 4, W4>(x, wt, st, zt, y, M, N, K, stream);
  const int64_t mid = (int64_t)((M + 255) / 256) * ((N + 127) / 128);
  if (mid >= 256) return launch_gemm<4, 2, W4>(x, wt, st, zt, y, M, N, K, stream);
  return launch_gemm<2, 2, W4>(x, wt, st, zt, y, M, N, K, stream);
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
