// Shared device helpers for the gfx950 kernels: 16-bit conversions, wave64 reductions,
// MFMA operand types, launch checking.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/olmo355.h"

typedef __bf16 bf16_t;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
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
template <> struct Act<O355_F16> {
  typedef uint16_t T;
  static __device__ __forceinline__ float ld(const void* p, int64_t i) { return (float)((const _Float16*)p)[i]; }
  static __device__ __forceinline__ void st(void* p, int64_t i, float v) { ((_Float16*)p)[i] = (_Float16)v; }
  static __device__ __forceinline__ float rnd(float v) { return (float)(_Float16)v; }
  static __device__ __forceinline__ float lowest() { return -65504.f; }
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
// A shuffle (`__shfl_xor`) compiles to a trip through the LDS crossbar that the wave waits out (ds_bpermute +
// s_waitcnt), six in a row for a butterfly over 64 lanes.  The same butterflies from register-to-register moves:
// DPP within rows of 16 lanes, v_permlane16_swap / v_permlane32_swap between half-rows and half-waves.  Operands and
// order of every step are those of the xor butterfly (after the xor-1 and xor-2 steps the lanes of a quad agree, so
// the mirrored partner of the next steps holds what the xor partner holds); the butterfly runs from distance 1 up
// to distance 32.
template <int CTRL>
__device__ __forceinline__ float dpp_lane(float v) {  // the value of the lane that DPP control CTRL names
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// op(v[l], v[l ^ 16]) in every lane (op commutative)
template <typename Op>
__device__ __forceinline__ float combine_xor16(float v, Op op) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);  // rows (0, 1) and (2, 3) trade places
  return op(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
// op(v[l], v[l ^ 32]) in every lane (op commutative)
template <typename Op>
__device__ __forceinline__ float combine_xor32(float v, Op op) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // the two halves of the wave
  return op(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
// reduction over an aligned row of 16 lanes; every lane gets it
template <typename Op>
__device__ __forceinline__ float row16_reduce(float v, Op op) {
  v = op(v, dpp_lane<0xB1>(v));   // quad_perm [1,0,3,2]
  v = op(v, dpp_lane<0x4E>(v));   // quad_perm [2,3,0,1]
  v = op(v, dpp_lane<0x141>(v));  // row_half_mirror
  v = op(v, dpp_lane<0x140>(v));  // row_mirror
  return v;
}
template <typename Op>
__device__ __forceinline__ float wave_reduce(float v, Op op) {
  return combine_xor32(combine_xor16(row16_reduce(v, op), op), op);
}
// one step of an xor butterfly, op(v[l], v[l ^ O]): register moves for the distances that have one (8: rotation of
// the row of 16 by 8; 16 and 32: the swaps above), a shuffle otherwise
template <int O, typename Op>
__device__ __forceinline__ float combine_xor(float v, Op op) {
  if constexpr (O == 32) return combine_xor32(v, op);
  else if constexpr (O == 16) return combine_xor16(v, op);
  else if constexpr (O == 8) return op(v, dpp_lane<0x128>(v));  // row_ror:8
  else if constexpr (O == 2) return op(v, dpp_lane<0x4E>(v));
  else if constexpr (O == 1) return op(v, dpp_lane<0xB1>(v));
  else return op(v, __shfl_xor(v, O, 64));
}
// The (value, index) pair that comes first under `before` (a strict total order: before(av, ai, bv, bi) = "a goes
// ahead of b") over the wave, in every lane.  DPP inside the rows of 16 lanes (after the first two steps a quad agrees,
// so the mirrored partner holds what the xor partner would), then the swaps between half-rows and half-waves, after
// which both candidates of a pair are at hand in every lane.
template <typename Before>
__device__ __forceinline__ void wave_first_pair(float& v, int& i, Before before) {
  auto take = [&](float ov, int oi) {
    if (before(ov, oi, v, i)) v = ov, i = oi;
  };
#define O355_PAIR_DPP(C) take(dpp_lane<C>(v), __builtin_amdgcn_update_dpp(0, i, C, 0xF, 0xF, true));
  O355_PAIR_DPP(0xB1)
  O355_PAIR_DPP(0x4E)
  O355_PAIR_DPP(0x141)
  O355_PAIR_DPP(0x140)
#undef O355_PAIR_DPP
  {
    const auto rv = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(uint32_t, v), __builtin_bit_cast(uint32_t, v), false, false);
    const auto ri = __builtin_amdgcn_permlane16_swap((uint32_t)i, (uint32_t)i, false, false);
    v = __builtin_bit_cast(float, (uint32_t)rv[0]), i = (int)ri[0];
    take(__builtin_bit_cast(float, (uint32_t)rv[1]), (int)ri[1]);
  }
  {
    const auto rv = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, v), __builtin_bit_cast(uint32_t, v), false, false);
    const auto ri = __builtin_amdgcn_permlane32_swap((uint32_t)i, (uint32_t)i, false, false);
    v = __builtin_bit_cast(float, (uint32_t)rv[0]), i = (int)ri[0];
    take(__builtin_bit_cast(float, (uint32_t)rv[1]), (int)ri[1]);
  }
}
struct AddOp { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };
struct MaxOp { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };

__device__ __forceinline__ float wave_sum(float v) { return wave_reduce(v, AddOp{}); }
__device__ __forceinline__ float wave_max(float v) { return wave_reduce(v, MaxOp{}); }
// sum over an aligned row of 16 lanes; every lane gets it
__device__ __forceinline__ float row16_sum(float v) { return row16_reduce(v, AddOp{}); }
// (kept under its older name: the wave sum has this form everywhere now)
__device__ __forceinline__ float wave_sum_dpp(float v) { return wave_sum(v); }

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

// The same word as 8 fp16 numbers for fp16 activations: fp16(scale * (q - zero)), the arithmetic of the reference's own
// dequantisation (qlinear_cuda_old.py:253-265: integer difference, one product, one rounding).  (1024 + q) - (1024 +
// zero) is exact in fp16, the product with the scale rounds once.
struct DequantConstsF16 {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  f16x2 s2, nz2;
};
__device__ __forceinline__ DequantConstsF16 dequant_consts_f16(uint16_t scale_bits, int zero) {
  const _Float16 s = __builtin_bit_cast(_Float16, scale_bits), nz = (_Float16)(-(float)(1024 + zero));
  return {{s, s}, {nz, nz}};
}
__device__ __forceinline__ u32x4 dequant_word_f16(uint32_t w, const DequantConstsF16& d) {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  u32x4 o;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const f16x2 h = __builtin_bit_cast(f16x2, ((w >> (4 * i)) & 0x000f000fu) | 0x64006400u);
    o[i] = __builtin_bit_cast(uint32_t, (f16x2)((h + d.nz2) * d.s2));
  }
  return o;
}
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {  // round to nearest even, as a cast does
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  const f16x2 p = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, p);
}

