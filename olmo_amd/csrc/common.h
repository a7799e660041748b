// Shared device helpers for the gfx950 kernels: 16-bit conversions, wave64 reductions,
// MFMA operand types, launch checking.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/olmo355.h"

typedef __bf16 bf16_t;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define O355_WAVE 64

#define O355_CHECK_LAUNCH()                       \
  do {                                            \
    hipError_t e__ = hipGetLastError();           \
    if (e__ != hipSuccess) return O355_ELAUNCH;   \
    return O355_OK;                               \
  } while (0)

static inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// int4 linear for 17..64 rows (gemv_mid.hip); arguments as olmo355_w4_gemv, already validated;
// pairs = column-tile pairs per workgroup (0 = choose)
int o355_w4_mid_dispatch(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                         int M, int N, int K, int pairs, void* stream);

// ---- scalar conversions -------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ float bf16lo_to_f32(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }
// round-to-nearest-even fp32 -> bf16 (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  bf16_t b = (bf16_t)f;
  return __builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2 p = {(bf16_t)lo, (bf16_t)hi};
  return __builtin_bit_cast(uint32_t, p);
}
__device__ __forceinline__ float round_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// Loads / stores of one activation element by dtype tag.
template <int DT> struct Act;
template <> struct Act<O355_F32> {
  typedef float T;
  static __device__ __forceinline__ float ld(const void* p, int64_t i) { return ((const float*)p)[i]; }
  static __device__ __forceinline__ void st(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
  static __device__ __forceinline__ float rnd(float v) { return v; }
  static __device__ __forceinline__ float lowest() { return -3.4028234663852886e38f; }
};
template <> struct Act<O355_BF16> {
  typedef uint16_t T;
  static __device__ __forceinline__ float ld(const void* p, int64_t i) {
    return bf16_bits_to_f32(((const uint16_t*)p)[i]);
  }
  static __device__ __forceinline__ void st(void* p, int64_t i, float v) { ((uint16_t*)p)[i] = f32_to_bf16_bits(v); }
  static __device__ __forceinline__ float rnd(float v) { return round_bf16(v); }
  static __device__ __forceinline__ float lowest() { return -3.3895313892515355e38f; }
};

// Workgroup barrier that orders LDS traffic only: global loads issued before it stay in flight
// (a plain __syncthreads() would wait for them as well).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---- buffer addressing ----------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// buffer resource over [base, base + bytes): loads past the end return zero
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, int64_t bytes) {
  const int64_t cap = 0xffffffffll;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)(uint32_t)(bytes < cap ? (bytes < 0 ? 0 : bytes) : cap),
                                           0x00020000);
}

// s_waitcnt immediate: at most `vm` vector-memory operations outstanding (and, with lds, no LDS ones)
constexpr int waitcnt_imm(int vm, bool lds) { return (vm & 15) | ((vm >> 4) << 14) | 0x0070 | (lds ? 0 : 0x0f00); }

// ---- wave64 reductions ------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// sum over an aligned row of 16 lanes; every lane gets it
__device__ __forceinline__ float row16_sum(float v) {
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, 16);
  return v;
}
// wave sum whose first four steps are DPP adds within rows of 16 lanes (fixed order: the same on every wave)
__device__ __forceinline__ float wave_sum_dpp(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // row_half_mirror
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // row_mirror
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}

// eight bf16 (one 16-byte piece) widened to fp32
__device__ __forceinline__ void unpack8(const u32x4& v, float (&f)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) f[2 * i] = bf16lo_to_f32(v[i]), f[2 * i + 1] = bf16hi_to_f32(v[i]);
}

// MFMA operand of eight ones: its product with the activations is their sum over k
__device__ __forceinline__ bf16x8 ones_bf16x8() {
  u32x4 r = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  return __builtin_bit_cast(bf16x8, r);
}

// Sum over the whole workgroup (blockDim.x a multiple of 64, at most 1024). `red` holds 16 floats.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}

// ---- int4 unpack -----------------------------------------------------------------------------
// The two constants of the unpack, made opaque to the optimiser (empty asm, no instruction): as
// literals the compiler emits v_and + v_or per pair, from registers it selects the single
// v_and_or_b32.  (An asm *instruction* here would be unsafe: the hazard recogniser does not see an
// asm's result feeding an MFMA and leaves out the wait states.)
struct UnpackConsts {
  uint32_t mask, bias;
  __device__ __forceinline__ UnpackConsts() : mask(0x000f000fu), bias(0x43004300u) {
    asm volatile("" : "+s"(mask));
    asm volatile("" : "+v"(bias));
  }
};

__device__ __forceinline__ bf16x8 unpack_w4_bias128(uint32_t w, const UnpackConsts& c) {
  u32x4 r;
  r.x = (w & c.mask) | c.bias;
  r.y = ((w >> 4) & c.mask) | c.bias;
  r.z = ((w >> 8) & c.mask) | c.bias;
  r.w = ((w >> 12) & c.mask) | c.bias;
  return __builtin_bit_cast(bf16x8, r);
}

