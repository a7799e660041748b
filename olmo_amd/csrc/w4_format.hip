// int4 group-wise weights: bit-exact fp16 dequantise table, one-time re-tiling into the
// MFMA-fragment layout, and the table read back from the tiled layout.
#include "common.h"

namespace {

__device__ __forceinline__ uint16_t dq_one(float s, int q, int z) {
  // exact fp32 product (11-bit x 5-bit significands), one RNE rounding to fp16, subnormals kept.
  // The sign is set explicitly: the compiler folds the multiply and the conversion into one
  // mixed-precision fma with a +0 addend, which would turn a -0 product (zero scale, q < zero)
  // into +0, and the table is compared bit for bit.
  const int d = q - z;
  _Float16 h = (_Float16)(s * (float)d);
  const uint16_t mag = __builtin_bit_cast(uint16_t, h) & 0x7fffu;
  const uint16_t sign = (uint16_t)(((__float_as_uint(s) >> 31) ^ (uint32_t)(d < 0)) << 15);
  return mag | sign;
}
__device__ __forceinline__ float h2f(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }

// one thread: one qweight word pair (row r, columns 2c, 2c+1) -> 8 rows x 2 columns of the table
__global__ __launch_bounds__(256) void w4_dequant_kernel(const int32_t* __restrict__ qweight,
                                                         const int32_t* __restrict__ qzeros,
                                                         const uint16_t* __restrict__ scales,
                                                         const int32_t* __restrict__ g_idx, uint32_t* __restrict__ out,
                                                         int K, int N, int group) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int half_n = N >> 1;
  const int64_t total = (int64_t)(K >> 3) * half_n;
  if (idx >= total) return;
  const int r = (int)(idx / half_n), c = (int)(idx % half_n);
  const int n0 = 2 * c;
  const uint32_t w0 = (uint32_t)qweight[(int64_t)r * N + n0], w1 = (uint32_t)qweight[(int64_t)r * N + n0 + 1];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int k = 8 * r + j;
    const int g = g_idx ? g_idx[k] : k / group;
    const uint32_t zw = (uint32_t)qzeros[(int64_t)g * (N >> 3) + (n0 >> 3)];
    const int z0 = (int)((zw >> (4 * (n0 & 7))) & 15u) + 1, z1 = (int)((zw >> (4 * ((n0 + 1) & 7))) & 15u) + 1;
    const float s0 = h2f(scales[(int64_t)g * N + n0]), s1 = h2f(scales[(int64_t)g * N + n0 + 1]);
    const int q0 = (int)((w0 >> (4 * j)) & 15u), q1 = (int)((w1 >> (4 * j)) & 15u);
    out[((int64_t)k * N + n0) >> 1] = (uint32_t)dq_one(s0, q0, z0) | ((uint32_t)dq_one(s1, q1, z1) << 16);
  }
}

// nibble order inside a tiled word: nibble p holds row offset e = 2p (p < 4) or 2(p-4)+1
__device__ __forceinline__ uint32_t nib_to_tiled(uint32_t w) {
  uint32_t o = 0;
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const int e = p < 4 ? 2 * p : 2 * (p - 4) + 1;
    o |= ((w >> (4 * e)) & 15u) << (4 * p);
  }
  return o;
}

// one thread per tiled word: (nt, g, lane, j)
__global__ __launch_bounds__(256) void w4_repack_kernel(const int32_t* __restrict__ qweight,
                                                        const int32_t* __restrict__ qzeros,
                                                        const uint16_t* __restrict__ scales, uint32_t* __restrict__ wt,
                                                        uint16_t* __restrict__ st, uint32_t* __restrict__ zt, int K,
                                                        int N) {
  const int G = K >> 7;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)(N >> 4) * G * 256;
  if (idx >= total) return;
  const int j = (int)(idx & 3), lane = (int)((idx >> 2) & 63);
  const int64_t tile = idx >> 8;
  const int g = (int)(tile % G), nt = (int)(tile / G);
  const int n = 16 * nt + (lane & 15);
  const int r = 16 * g + 4 * j + (lane >> 4);
  wt[idx] = nib_to_tiled((uint32_t)qweight[(int64_t)r * N + n]);
  if (j == 0 && lane < 16) st[tile * 16 + lane] = scales[(int64_t)g * N + 16 * nt + lane];
  if (j == 0 && lane >= 16 && lane < 18)
    zt[tile * 2 + (lane - 16)] = (uint32_t)qzeros[(int64_t)g * (N >> 3) + 2 * nt + (lane - 16)];
}

__global__ __launch_bounds__(256) void w4t_dequant_kernel(const uint32_t* __restrict__ wt,
                                                          const uint16_t* __restrict__ st,
                                                          const uint8_t* __restrict__ zt, uint16_t* __restrict__ out,
                                                          int K, int N) {
  const int G = K >> 7;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)(N >> 4) * G * 256;
  if (idx >= total) return;
  const int j = (int)(idx & 3), lane = (int)((idx >> 2) & 63);
  const int64_t tile = idx >> 8;
  const int g = (int)(tile % G), nt = (int)(tile / G);
  const int c = lane & 15;
  const int n = 16 * nt + c;
  const uint32_t w = wt[idx];
  const float s = h2f(st[tile * 16 + c]);
  const int z = (int)((zt[tile * 8 + (c >> 1)] >> (4 * (c & 1))) & 15u) + 1;
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const int e = p < 4 ? 2 * p : 2 * (p - 4) + 1;
    const int k = 128 * g + 32 * j + 8 * (lane >> 4) + e;
    out[(int64_t)k * N + n] = dq_one(s, (int)((w >> (4 * p)) & 15u), z);
  }
}

}  // namespace

extern "C" int olmo355_w4_dequant_fp16(const int32_t* qweight, const int32_t* qzeros, const uint16_t* scales,
                                       const int32_t* g_idx, uint16_t* out_kn, int K, int N, int group,
                                       void* stream) {
  if (!qweight || !qzeros || !scales || !out_kn) return O355_EINVAL;
  if (K <= 0 || N <= 0 || (K & 7) || (N & 7)) return O355_EINVAL;
  if (!g_idx && (group <= 0 || K % group)) return O355_EINVAL;
  const int64_t total = (int64_t)(K >> 3) * (N >> 1);
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipLaunchKernelGGL(w4_dequant_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), qweight, qzeros, scales, g_idx,
                     (uint32_t*)out_kn, K, N, group);
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_w4_repack(const int32_t* qweight, const int32_t* qzeros, const uint16_t* scales, uint32_t* wt,
                                 uint16_t* st, uint8_t* zt, int K, int N, int group, void* stream) {
  if (!qweight || !qzeros || !scales || !wt || !st || !zt) return O355_EINVAL;
  if (K <= 0 || N <= 0) return O355_EINVAL;
  if (group != 128 || (K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  const int64_t total = (int64_t)(N >> 4) * (K >> 7) * 256;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipLaunchKernelGGL(w4_repack_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), qweight, qzeros, scales, wt, st,
                     (uint32_t*)zt, K, N);
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_w4t_dequant_fp16(const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* out_kn,
                                        int K, int N, void* stream) {
  if (!wt || !st || !zt || !out_kn) return O355_EINVAL;
  if (K <= 0 || N <= 0) return O355_EINVAL;
  if ((K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  const int64_t total = (int64_t)(N >> 4) * (K >> 7) * 256;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipLaunchKernelGGL(w4t_dequant_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), wt, st, zt, out_kn, K, N);
  O355_CHECK_LAUNCH();
}
