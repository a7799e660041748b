// Bandwidth-bound row kernels: RMSNorm (+ residual add), non-parametric LayerNorm, QK-norm +
// rotary + KV-cache write, SwiGLU, embedding lookup, residual add, argmax.
// Rounding points follow the reference op by op so that a 16-bit activation dtype gives the
// same values as the reference's eager op chains.
//
// Rows are read once with 16-byte loads and kept in registers between the reduction and the
// normalisation pass (a decode step has one row per sequence, so these kernels are pure
// latency: every load of a row is issued before the first use).
#include "common.h"
#include <type_traits>

namespace {

// 16 bytes of activations as floats: 8 bf16 or 4 fp32.
template <int DT> struct Vec;
template <> struct Vec<O355_BF16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void ld(const void* p, int64_t vec_idx, float (&f)[8]) {
    const u32x4 v = reinterpret_cast<const u32x4*>(p)[vec_idx];
#pragma unroll
    for (int i = 0; i < 4; ++i) f[2 * i] = bf16lo_to_f32(v[i]), f[2 * i + 1] = bf16hi_to_f32(v[i]);
  }
  static __device__ __forceinline__ void st(void* p, int64_t vec_idx, const float (&f)[8]) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = pack_bf16x2(f[2 * i], f[2 * i + 1]);
    reinterpret_cast<u32x4*>(p)[vec_idx] = v;
  }
};
template <> struct Vec<O355_F16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void ld(const void* p, int64_t vec_idx, float (&f)[8]) {
    const u32x4 v = reinterpret_cast<const u32x4*>(p)[vec_idx];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f16x2 h = __builtin_bit_cast(f16x2, (uint32_t)v[i]);
      f[2 * i] = (float)h[0], f[2 * i + 1] = (float)h[1];
    }
  }
  static __device__ __forceinline__ void st(void* p, int64_t vec_idx, const float (&f)[8]) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = pack_f16x2(f[2 * i], f[2 * i + 1]);
    reinterpret_cast<u32x4*>(p)[vec_idx] = v;
  }
};
template <> struct Vec<O355_F32> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void ld(const void* p, int64_t vec_idx, float (&f)[4]) {
    const f32x4 v = reinterpret_cast<const f32x4*>(p)[vec_idx];
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = v[i];
  }
  static __device__ __forceinline__ void st(void* p, int64_t vec_idx, const float (&f)[4]) {
    f32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = f[i];
    reinterpret_cast<f32x4*>(p)[vec_idx] = v;
  }
};

// ---- RMSNorm: olmo/model.py:241-255 ---------------------------------------------------------------
// fp32 normalise -> round to dtype -> multiply by weight in dtype (second rounding) -> optional
// residual add in dtype (third rounding).  VPT vectors per thread held in registers.
template <int DT, int VPT>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(const void* __restrict__ x, const void* __restrict__ w,
                                                          const void* __restrict__ res, void* __restrict__ out, int d,
                                                          float eps) {
  constexpr int N = Vec<DT>::N;
  __shared__ float red[16];
  const int nvec = d / N;
  const int64_t vbase = (int64_t)blockIdx.x * nvec;
  float v[VPT][N];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec) Vec<DT>::ld(x, vbase + idx, v[i]);
  }
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec) {
#pragma unroll
      for (int e = 0; e < N; ++e) ss += v[i][e] * v[i][e];
    }
  }
  ss = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(ss / (float)d + eps);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec) {
      float wv[N], rv[N];
      if (w) Vec<DT>::ld(w, idx, wv);
      if (res) Vec<DT>::ld(res, vbase + idx, rv);
#pragma unroll
      for (int e = 0; e < N; ++e) {
        float y = Act<DT>::rnd(v[i][e] * rstd);
        if (w) y = Act<DT>::rnd(wv[e] * y);
        if (res) y = rv[e] + y;
        v[i][e] = y;
      }
      Vec<DT>::st(out, vbase + idx, v[i]);
    }
  }
}

// Two norms in one launch, for the end of a decode step: x1 = res + rmsnorm(x; w1), out = rmsnorm(x1; w2), every
// rounding where the two separate launches have it (x1 is rounded to the activation type before its squares are summed).
template <int DT, int VPT>
__global__ __launch_bounds__(256) void rmsnorm_pair_kernel(const void* __restrict__ x, const void* __restrict__ w1,
                                                           const void* __restrict__ res, const void* __restrict__ w2,
                                                           void* __restrict__ out, int d, float eps) {
  constexpr int N = Vec<DT>::N;
  __shared__ float red[16];
  const int nvec = d / N;
  const int64_t vbase = (int64_t)blockIdx.x * nvec;
  float v[VPT][N];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec) {
      Vec<DT>::ld(x, vbase + idx, v[i]);
#pragma unroll
      for (int e = 0; e < N; ++e) ss += v[i][e] * v[i][e];
    }
  }
  ss = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(ss / (float)d + eps);
  float ss2 = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec) {
      float wv[N], rv[N];
      Vec<DT>::ld(w1, idx, wv);
      Vec<DT>::ld(res, vbase + idx, rv);
#pragma unroll
      for (int e = 0; e < N; ++e) {
        const float y = Act<DT>::rnd(wv[e] * Act<DT>::rnd(v[i][e] * rstd));
        v[i][e] = Act<DT>::rnd(rv[e] + y);
        ss2 += v[i][e] * v[i][e];
      }
    }
  }
  ss2 = block_sum(ss2, red);
  const float rstd2 = 1.f / sqrtf(ss2 / (float)d + eps);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = threadIdx.x + i * 256;
    if (idx < nvec) {
      float wv[N];
      Vec<DT>::ld(w2, idx, wv);
#pragma unroll
      for (int e = 0; e < N; ++e) v[i][e] = Act<DT>::rnd(wv[e] * Act<DT>::rnd(v[i][e] * rstd2));
      Vec<DT>::st(out, vbase + idx, v[i]);
    }
  }
}

// any d (element-wise fallback)
template <int DT>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const void* __restrict__ x, const void* __restrict__ w,
                                                      const void* __restrict__ res, void* __restrict__ out, int d,
                                                      float eps) {
  __shared__ float red[16];
  const int64_t base = (int64_t)blockIdx.x * d;
  float ss = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const float v = Act<DT>::ld(x, base + i);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(ss / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float v = Act<DT>::rnd(Act<DT>::ld(x, base + i) * rstd);
    if (w) v = Act<DT>::rnd(Act<DT>::ld(w, i) * v);
    if (res) v = Act<DT>::ld(res, base + i) + v;
    Act<DT>::st(out, base + i, v);
  }
}

// ---- non-parametric LayerNorm: olmo/model.py:212-225 (F.layer_norm, biased variance) ------------------
template <int DT>
__global__ __launch_bounds__(256) void layernorm_np_kernel(const void* __restrict__ x, void* __restrict__ out, int d,
                                                           float eps) {
  __shared__ float red[16];
  const int64_t base = (int64_t)blockIdx.x * d;
  float s = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) s += Act<DT>::ld(x, base + i);
  const float mean = block_sum(s, red) / (float)d;
  float v2 = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const float c = Act<DT>::ld(x, base + i) - mean;
    v2 += c * c;
  }
  const float var = block_sum(v2, red) / (float)d;
  const float rstd = 1.f / sqrtf(var + eps);
  for (int i = threadIdx.x; i < d; i += blockDim.x)
    Act<DT>::st(out, base + i, (Act<DT>::ld(x, base + i) - mean) * rstd);
}

// ---- QK-norm + rotary + cache write ----------------------------------------------------------------
// One workgroup per token row.  olmo/model.py:603-605 (norm over the *whole* q / k width),
// :298-324 (rotate_half convention, fp32 math: t*cos + rot*sin, each product rounded),
// :615-620 (cache append).
//
// Vector form (bf16, hd % 16 == 0): a thread owns "pair chunks" -- 8 channels j..j+7 of the first
// half of a head and the 8 channels j+hd/2.. they rotate with.  CPT chunks per thread for q and
// for k stay in registers across the sum-of-squares reduction.
template <int CPT>
__global__ __launch_bounds__(256) void qknorm_rope_vec_kernel(const uint16_t* __restrict__ qkv,
                                                              const uint16_t* __restrict__ qw,
                                                              const uint16_t* __restrict__ kw,
                                                              const float* __restrict__ sin_t,
                                                              const float* __restrict__ cos_t, uint16_t* __restrict__ q_out,
                                                              uint16_t* __restrict__ kc, uint16_t* __restrict__ vc, int T,
                                                              int H, int Hkv, int hd, int Lmax, int n_pos, int past_len,
                                                              const int32_t* __restrict__ past_dev, float eps) {
  constexpr int DT = O355_BF16;
  __shared__ float red[16];
  const int row = blockIdx.x, b = row / T, t = row % T;
  const int dq = H * hd, dk = Hkv * hd, half = hd >> 1, cph = hd >> 4;  // chunks per head
  const int64_t in_base = (int64_t)row * (dq + 2 * dk);
  const int pos = (past_dev ? *past_dev : past_len) + t;
  if (pos >= Lmax || pos >= n_pos) return;  // a device-side position beyond the cache: write nothing
  const bool norm = (qw != nullptr);
  const int nq = H * cph, nk = Hkv * cph;

  float q1[CPT][8], q2[CPT][8], k1[CPT][8], k2[CPT][8];
  float sq = 0.f, sk = 0.f;
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < nq) {
      const int64_t e = in_base + (c / cph) * hd + (c % cph) * 8;
      Vec<DT>::ld(qkv, e >> 3, q1[i]);
      Vec<DT>::ld(qkv, (e + half) >> 3, q2[i]);
    }
    if (c < nk) {
      const int64_t e = in_base + dq + (c / cph) * hd + (c % cph) * 8;
      Vec<DT>::ld(qkv, e >> 3, k1[i]);
      Vec<DT>::ld(qkv, (e + half) >> 3, k2[i]);
    }
  }
  // v: straight copy into the cache
  for (int c = threadIdx.x; c < (dk >> 3); c += 256) {
    const int h = (c * 8) / hd, j = (c * 8) % hd;
    const u32x4 v = reinterpret_cast<const u32x4*>(qkv)[(in_base + dq + dk + c * 8) >> 3];
    reinterpret_cast<u32x4*>(vc)[((((int64_t)b * Hkv + h) * Lmax + pos) * hd + j) >> 3] = v;
  }
  float rq = 1.f, rk = 1.f;
  if (norm) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = threadIdx.x + i * 256;
      if (c < nq) {
#pragma unroll
        for (int e = 0; e < 8; ++e) sq += q1[i][e] * q1[i][e] + q2[i][e] * q2[i][e];
      }
      if (c < nk) {
#pragma unroll
        for (int e = 0; e < 8; ++e) sk += k1[i][e] * k1[i][e] + k2[i][e] * k2[i][e];
      }
    }
    rq = 1.f / sqrtf(block_sum(sq, red) / (float)dq + eps);
    rk = 1.f / sqrtf(block_sum(sk, red) / (float)dk + eps);
  }
  const float* sn = sin_t + (int64_t)pos * hd;
  const float* cs = cos_t + (int64_t)pos * hd;
  auto rotate = [&](float (&x1)[8], float (&x2)[8], const uint16_t* wgt, int ch, float r, int j) {
    // ch: channel index of x1[0] inside the q (or k) vector; j: its index inside the head
    float w1[8], w2[8], c1[8], c2[8], s1[8], s2[8];
    if (norm) {
      Vec<DT>::ld(wgt, ch >> 3, w1);
      Vec<DT>::ld(wgt, (ch + half) >> 3, w2);
    }
#pragma unroll
    for (int v4 = 0; v4 < 2; ++v4) {  // table rows are 16-byte aligned: hd % 16 == 0, j % 8 == 0
      const f32x4 a1 = reinterpret_cast<const f32x4*>(cs + j)[v4], a2 = reinterpret_cast<const f32x4*>(cs + j + half)[v4];
      const f32x4 b1 = reinterpret_cast<const f32x4*>(sn + j)[v4], b2 = reinterpret_cast<const f32x4*>(sn + j + half)[v4];
#pragma unroll
      for (int e = 0; e < 4; ++e) c1[4 * v4 + e] = a1[e], c2[4 * v4 + e] = a2[e], s1[4 * v4 + e] = b1[e], s2[4 * v4 + e] = b2[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float a = x1[e], bb = x2[e];
      if (norm) {
        a = Act<DT>::rnd(w1[e] * Act<DT>::rnd(a * r));
        bb = Act<DT>::rnd(w2[e] * Act<DT>::rnd(bb * r));
      }
      x1[e] = __fadd_rn(__fmul_rn(a, c1[e]), __fmul_rn(-bb, s1[e]));
      x2[e] = __fadd_rn(__fmul_rn(bb, c2[e]), __fmul_rn(a, s2[e]));
    }
  };
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < nq) {
      const int h = c / cph, j = (c % cph) * 8;
      rotate(q1[i], q2[i], qw, h * hd + j, rq, j);
      const int64_t o = (int64_t)row * dq + h * hd + j;
      Vec<DT>::st(q_out, o >> 3, q1[i]);
      Vec<DT>::st(q_out, (o + half) >> 3, q2[i]);
    }
    if (c < nk) {
      const int h = c / cph, j = (c % cph) * 8;
      rotate(k1[i], k2[i], kw, h * hd + j, rk, j);
      const int64_t o = (((int64_t)b * Hkv + h) * Lmax + pos) * hd + j;
      Vec<DT>::st(kc, o >> 3, k1[i]);
      Vec<DT>::st(kc, (o + half) >> 3, k2[i]);
    }
  }
}

// any dtype / head size (element-wise)
template <int DT>
__global__ __launch_bounds__(256) void qknorm_rope_kernel(const void* __restrict__ qkv, const void* __restrict__ qw,
                                                          const void* __restrict__ kw, const float* __restrict__ sin_t,
                                                          const float* __restrict__ cos_t, void* __restrict__ q_out,
                                                          void* __restrict__ kc, void* __restrict__ vc, int T, int H,
                                                          int Hkv, int hd, int Lmax, int n_pos, int past_len,
                                                          const int32_t* __restrict__ past_dev, float eps) {
  __shared__ float red[16];
  const int row = blockIdx.x;  // b*T + t
  const int b = row / T, t = row % T;
  const int dq = H * hd, dk = Hkv * hd;
  const int64_t in_base = (int64_t)row * (dq + 2 * dk);
  const int past = past_dev ? *past_dev : past_len;
  const int pos = past + t;
  if (pos >= Lmax || pos >= n_pos) return;  // a device-side position beyond the cache: write nothing
  const bool norm = (qw != nullptr);

  float rq = 1.f, rk = 1.f;
  if (norm) {
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < dq; i += blockDim.x) {
      const float v = Act<DT>::ld(qkv, in_base + i);
      sq += v * v;
    }
    for (int i = threadIdx.x; i < dk; i += blockDim.x) {
      const float v = Act<DT>::ld(qkv, in_base + dq + i);
      sk += v * v;
    }
    rq = 1.f / sqrtf(block_sum(sq, red) / (float)dq + eps);
    rk = 1.f / sqrtf(block_sum(sk, red) / (float)dk + eps);
  }
  const int half = hd >> 1;
  const float* sn = sin_t + (int64_t)pos * hd;
  const float* cs = cos_t + (int64_t)pos * hd;
  for (int p = threadIdx.x; p < H * half; p += blockDim.x) {
    const int h = p / half, j = p % half;
    const int i1 = h * hd + j, i2 = i1 + half;
    float x1 = Act<DT>::ld(qkv, in_base + i1), x2 = Act<DT>::ld(qkv, in_base + i2);
    if (norm) {
      x1 = Act<DT>::rnd(Act<DT>::ld(qw, i1) * Act<DT>::rnd(x1 * rq));
      x2 = Act<DT>::rnd(Act<DT>::ld(qw, i2) * Act<DT>::rnd(x2 * rq));
    }
    const float o1 = __fadd_rn(__fmul_rn(x1, cs[j]), __fmul_rn(-x2, sn[j]));
    const float o2 = __fadd_rn(__fmul_rn(x2, cs[j + half]), __fmul_rn(x1, sn[j + half]));
    Act<DT>::st(q_out, (int64_t)row * dq + i1, o1);
    Act<DT>::st(q_out, (int64_t)row * dq + i2, o2);
  }
  for (int p = threadIdx.x; p < Hkv * half; p += blockDim.x) {
    const int h = p / half, j = p % half;
    const int i1 = h * hd + j, i2 = i1 + half;
    float x1 = Act<DT>::ld(qkv, in_base + dq + i1), x2 = Act<DT>::ld(qkv, in_base + dq + i2);
    if (norm) {
      x1 = Act<DT>::rnd(Act<DT>::ld(kw, i1) * Act<DT>::rnd(x1 * rk));
      x2 = Act<DT>::rnd(Act<DT>::ld(kw, i2) * Act<DT>::rnd(x2 * rk));
    }
    const float o1 = __fadd_rn(__fmul_rn(x1, cs[j]), __fmul_rn(-x2, sn[j]));
    const float o2 = __fadd_rn(__fmul_rn(x2, cs[j + half]), __fmul_rn(x1, sn[j + half]));
    const int64_t cb = (((int64_t)b * Hkv + h) * Lmax + pos) * hd;
    Act<DT>::st(kc, cb + j, o1);
    Act<DT>::st(kc, cb + j + half, o2);
  }
  for (int i = threadIdx.x; i < dk; i += blockDim.x) {
    const int h = i / hd, j = i % hd;
    const int64_t cb = (((int64_t)b * Hkv + h) * Lmax + pos) * hd;
    Act<DT>::st(vc, cb + j, Act<DT>::ld(qkv, in_base + dq + dk + i));
  }
}

// ---- SwiGLU: olmo/model.py:365-368 -----------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void swiglu_kernel(const void* __restrict__ x, void* __restrict__ out, int64_t total,
                                                     int h) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int64_t r = idx / h;
  const int c = (int)(idx % h);
  const float up = Act<DT>::ld(x, r * 2 * h + c), gate = Act<DT>::ld(x, r * 2 * h + h + c);
  const float s = Act<DT>::rnd(gate / (1.f + expf(-gate)));
  Act<DT>::st(out, idx, s * up);
}

// h % Vec::N == 0: one 16-byte piece of up and of gate per thread
template <int DT>
__global__ __launch_bounds__(256) void swiglu_vec_kernel(const void* __restrict__ x, void* __restrict__ out,
                                                         int64_t total_vec, int hv) {
  constexpr int N = Vec<DT>::N;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total_vec) return;
  const int64_t r = idx / hv;
  const int c = (int)(idx % hv);
  float up[N], gate[N];
  Vec<DT>::ld(x, r * 2 * hv + c, up);
  Vec<DT>::ld(x, r * 2 * hv + hv + c, gate);
#pragma unroll
  for (int e = 0; e < N; ++e) up[e] = Act<DT>::rnd(gate[e] / (1.f + expf(-gate[e]))) * up[e];
  Vec<DT>::st(out, idx, up);
}

template <int DT>
__global__ __launch_bounds__(256) void embedding_kernel(const int64_t* __restrict__ ids, const void* __restrict__ tab,
                                                        void* __restrict__ out, int d, int vocab) {
  int64_t id = ids[blockIdx.x];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  typedef typename Act<DT>::T T;
  const T* src = (const T*)tab + id * d;
  T* dst = (T*)out + (int64_t)blockIdx.x * d;
  if (((d * sizeof(T)) & 15) == 0) {
    const int nv = (int)(d * sizeof(T) / 16);
    for (int i = threadIdx.x; i < nv; i += blockDim.x)
      reinterpret_cast<u32x4*>(dst)[i] = reinterpret_cast<const u32x4*>(src)[i];
  } else {
    for (int i = threadIdx.x; i < d; i += blockDim.x) dst[i] = src[i];
  }
}

template <int DT>
__global__ __launch_bounds__(256) void add_kernel(const void* __restrict__ a, const void* __restrict__ b,
                                                  void* __restrict__ out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) Act<DT>::st(out, i, Act<DT>::ld(a, i) + Act<DT>::ld(b, i));
}

// out[m][n] = x[m][n] + bias[n], bias fp16 (the QuantLinear bias buffer), sum in fp32, one rounding
__global__ __launch_bounds__(256) void add_bias_bf16_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ bias,
                                                            uint16_t* __restrict__ out, int64_t total, int N) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) {
    const float b = (float)__builtin_bit_cast(_Float16, bias[i % N]);
    out[i] = (uint16_t)f32_to_bf16_bits(bf16_bits_to_f32(x[i]) + b);
  }
}

// the same for fp16 rows (QuantLinear.forward on fp16 input: out + bias, qlinear_cuda_old.py:288-290)
__global__ __launch_bounds__(256) void add_bias_f16_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ bias,
                                                           uint16_t* __restrict__ out, int64_t total, int N) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) {
    const float b = (float)__builtin_bit_cast(_Float16, bias[i % N]);
    out[i] = __builtin_bit_cast(uint16_t, (_Float16)((float)__builtin_bit_cast(_Float16, x[i]) + b));
  }
}

// first index of the maximum of each row (torch.argmax tie rule); all loads of a thread issued
// up front when the row is 16-byte divisible
template <int DT>
__global__ __launch_bounds__(1024) void argmax_kernel(const void* __restrict__ x, int64_t* __restrict__ out, int n) {
  constexpr int N = Vec<DT>::N;
  constexpr int VPT = 16;
  __shared__ float sv[16];
  __shared__ int si[16];
  const int64_t base = (int64_t)blockIdx.x * n;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  if (n % N == 0 && n / N <= VPT * 1024) {
    const int nvec = n / N;
    float v[VPT][N];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int idx = threadIdx.x + i * 1024;
      if (idx < nvec) Vec<DT>::ld(x, (base / N) + idx, v[i]);
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int idx = threadIdx.x + i * 1024;
      if (idx < nvec) {
#pragma unroll
        for (int e = 0; e < N; ++e)
          if (v[i][e] > best) best = v[i][e], bi = idx * N + e;  // indices ascend per thread: first max kept
      }
    }
  } else {
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const float v = Act<DT>::ld(x, base + i);
      if (v > best || (v == best && i < bi)) best = v, bi = i;
    }
  }
  // the wave's winner: largest value, smallest index among equals
  wave_first_pair(best, bi, [](float ov, int oi, float v, int i) { return ov > v || (ov == v && oi < i); });
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) sv[w] = best, si[w] = bi;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i)
      if (sv[i] > best || (sv[i] == best && si[i] < bi)) best = sv[i], bi = si[i];
    out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
  }
}

// The end of a greedy decode step in one launch: argmax_kernel's choice per row, the chosen token's embedding row as
// the next step's input, and (row 0's workgroup) the position advanced by one with its rotary rows, as
// olmo355_rope_advance leaves them.
template <int DT>
__global__ __launch_bounds__(1024) void greedy_next_kernel(const void* __restrict__ x, int64_t* __restrict__ out, int n,
                                                           const void* __restrict__ tab, void* __restrict__ x_next, int d,
                                                           int vocab, int32_t* __restrict__ pos,
                                                           const float* __restrict__ sin_t, const float* __restrict__ cos_t,
                                                           float* __restrict__ rope_now, int hd, int n_pos) {
  constexpr int N = Vec<DT>::N;
  constexpr int VPT = 16;
  __shared__ float sv[16];
  __shared__ int si[16];
  const int64_t base = (int64_t)blockIdx.x * n;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  if (n % N == 0 && n / N <= VPT * 1024) {
    const int nvec = n / N;
    float v[VPT][N];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int idx = threadIdx.x + i * 1024;
      if (idx < nvec) Vec<DT>::ld(x, (base / N) + idx, v[i]);
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int idx = threadIdx.x + i * 1024;
      if (idx < nvec) {
#pragma unroll
        for (int e = 0; e < N; ++e)
          if (v[i][e] > best) best = v[i][e], bi = idx * N + e;  // indices ascend per thread: first max kept
      }
    }
  } else {
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const float v = Act<DT>::ld(x, base + i);
      if (v > best || (v == best && i < bi)) best = v, bi = i;
    }
  }
  wave_first_pair(best, bi, [](float ov, int oi, float v, int i) { return ov > v || (ov == v && oi < i); });
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) sv[w] = best, si[w] = bi;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i)
      if (sv[i] > best || (sv[i] == best && si[i] < bi)) best = sv[i], bi = si[i];
    bi = bi == 0x7fffffff ? 0 : bi;
    out[blockIdx.x] = bi;
    si[0] = bi;
  }
  __syncthreads();
  // the chosen token's row of the embedding table (clamped like embedding_kernel's)
  int64_t id = si[0];
  id = id >= vocab ? vocab - 1 : id;
  typedef typename Act<DT>::T T;
  const T* src = (const T*)tab + id * d;
  T* dst = (T*)x_next + (int64_t)blockIdx.x * d;
  if (((d * sizeof(T)) & 15) == 0) {
    const int nv = (int)(d * sizeof(T) / 16);
    for (int i = threadIdx.x; i < nv; i += blockDim.x) reinterpret_cast<u32x4*>(dst)[i] = reinterpret_cast<const u32x4*>(src)[i];
  } else {
    for (int i = threadIdx.x; i < d; i += blockDim.x) dst[i] = src[i];
  }
  if (blockIdx.x == 0) {
    const int p = *pos + 1;
    __syncthreads();  // every thread has read the old value
    if (threadIdx.x == 0) *pos = p;
    const int r = min(max(p, 0), n_pos - 1);
    for (int i = threadIdx.x; i < hd; i += blockDim.x) {
      rope_now[i] = sin_t[(int64_t)r * hd + i];
      rope_now[hd + i] = cos_t[(int64_t)r * hd + i];
    }
  }
}

__global__ void incr_kernel(int32_t* p) { *p += 1; }

}  // namespace

#define DT_SWITCH(dtype, ...)                               \
  if ((dtype) == O355_F32) {                                \
    constexpr int DT = O355_F32;                            \
    __VA_ARGS__;                                            \
  } else if ((dtype) == O355_BF16) {                        \
    constexpr int DT = O355_BF16;                           \
    __VA_ARGS__;                                            \
  } else if ((dtype) == O355_F16) {                         \
    constexpr int DT = O355_F16;                            \
    __VA_ARGS__;                                            \
  } else {                                                  \
    return O355_EUNSUPPORTED;                               \
  }

extern "C" int olmo355_rmsnorm(const void* x, const void* weight, const void* residual, void* out, int rows, int d,
                               float eps, int dtype, void* stream) {
  if (!x || !out || rows <= 0 || d <= 0) return O355_EINVAL;
  hipStream_t s = as_stream(stream);
  const int vn = dtype == O355_F32 ? 4 : 8;
  const int nvec = d / vn;
  if (d % vn == 0 && nvec <= 4 * 256) {
    if (nvec <= 256) {
      DT_SWITCH(dtype, hipLaunchKernelGGL((rmsnorm_vec_kernel<DT, 1>), dim3(rows), dim3(256), 0, s, x, weight, residual,
                                          out, d, eps));
    } else if (nvec <= 512) {
      DT_SWITCH(dtype, hipLaunchKernelGGL((rmsnorm_vec_kernel<DT, 2>), dim3(rows), dim3(256), 0, s, x, weight, residual,
                                          out, d, eps));
    } else {
      DT_SWITCH(dtype, hipLaunchKernelGGL((rmsnorm_vec_kernel<DT, 4>), dim3(rows), dim3(256), 0, s, x, weight, residual,
                                          out, d, eps));
    }
  } else {
    DT_SWITCH(dtype,
              hipLaunchKernelGGL(rmsnorm_kernel<DT>, dim3(rows), dim3(256), 0, s, x, weight, residual, out, d, eps));
  }
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_rmsnorm_pair(const void* x, const void* w1, const void* residual, const void* w2, void* out,
                                    int rows, int d, float eps, int dtype, void* stream) {
  if (!x || !w1 || !residual || !w2 || !out || rows <= 0 || d <= 0) return O355_EINVAL;
  hipStream_t s = as_stream(stream);
  const int vn = dtype == O355_F32 ? 4 : 8;
  const int nvec = d / vn;
  if (d % vn != 0 || nvec > 4 * 256) return O355_EUNSUPPORTED;  // the caller issues the two norms one after the other
  if (nvec <= 256) {
    DT_SWITCH(dtype, hipLaunchKernelGGL((rmsnorm_pair_kernel<DT, 1>), dim3(rows), dim3(256), 0, s, x, w1, residual, w2, out, d, eps));
  } else if (nvec <= 512) {
    DT_SWITCH(dtype, hipLaunchKernelGGL((rmsnorm_pair_kernel<DT, 2>), dim3(rows), dim3(256), 0, s, x, w1, residual, w2, out, d, eps));
  } else {
    DT_SWITCH(dtype, hipLaunchKernelGGL((rmsnorm_pair_kernel<DT, 4>), dim3(rows), dim3(256), 0, s, x, w1, residual, w2, out, d, eps));
  }
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_layernorm_np(const void* x, void* out, int rows, int d, float eps, int dtype, void* stream) {
  if (!x || !out || rows <= 0 || d <= 0) return O355_EINVAL;
  DT_SWITCH(dtype,
            hipLaunchKernelGGL(layernorm_np_kernel<DT>, dim3(rows), dim3(256), 0, as_stream(stream), x, out, d, eps));
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_qknorm_rope_kvwrite(const void* qkv, const void* qw, const void* kw, const float* sin_tab,
                                           const float* cos_tab, void* q_out, void* kcache, void* vcache, int B, int T,
                                           int H, int Hkv, int hd, int Lmax, int n_pos, int past_len,
                                           const int32_t* past_len_dev, float eps, int dtype, void* stream) {
  if (!qkv || !sin_tab || !cos_tab || !q_out || !kcache || !vcache) return O355_EINVAL;
  if (B <= 0 || T <= 0 || H <= 0 || Hkv <= 0 || hd <= 0 || (hd & 1) || Lmax <= 0 || past_len < 0) return O355_EINVAL;
  if ((qw == nullptr) != (kw == nullptr)) return O355_EINVAL;
  if (!past_len_dev && (past_len + T > Lmax || past_len + T > n_pos)) return O355_EINVAL;
  if (past_len_dev && T != 1) return O355_EUNSUPPORTED;
  hipStream_t s = as_stream(stream);
  const int chunks = (H * hd) >> 4;
  if (dtype == O355_BF16 && (hd & 15) == 0 && chunks <= 4 * 256) {
#define QK_VEC(CPT)                                                                                                 \
  hipLaunchKernelGGL(qknorm_rope_vec_kernel<CPT>, dim3(B * T), dim3(256), 0, s, (const uint16_t*)qkv,              \
                     (const uint16_t*)qw, (const uint16_t*)kw, sin_tab, cos_tab, (uint16_t*)q_out, (uint16_t*)kcache, \
                     (uint16_t*)vcache, T, H, Hkv, hd, Lmax, n_pos, past_len, past_len_dev, eps)
    if (chunks <= 256) QK_VEC(1);
    else if (chunks <= 512) QK_VEC(2);
    else QK_VEC(4);
#undef QK_VEC
    O355_CHECK_LAUNCH();
  }
  DT_SWITCH(dtype, hipLaunchKernelGGL(qknorm_rope_kernel<DT>, dim3(B * T), dim3(256), 0, s, qkv, qw, kw, sin_tab,
                                      cos_tab, q_out, kcache, vcache, T, H, Hkv, hd, Lmax, n_pos, past_len, past_len_dev,
                                      eps));
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_swiglu(const void* x, void* out, int rows, int h, int dtype, void* stream) {
  if (!x || !out || rows <= 0 || h <= 0) return O355_EINVAL;
  const int vn = dtype == O355_F32 ? 4 : 8;
  if (h % vn == 0) {
    const int64_t total = (int64_t)rows * (h / vn);
    DT_SWITCH(dtype, hipLaunchKernelGGL(swiglu_vec_kernel<DT>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                                        as_stream(stream), x, out, total, h / vn));
  } else {
    const int64_t total = (int64_t)rows * h;
    DT_SWITCH(dtype, hipLaunchKernelGGL(swiglu_kernel<DT>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                                        as_stream(stream), x, out, total, h));
  }
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_embedding(const int64_t* ids, const void* table, void* out, int rows, int d, int vocab,
                                 int dtype, void* stream) {
  if (!ids || !table || !out || rows <= 0 || d <= 0 || vocab <= 0) return O355_EINVAL;
  DT_SWITCH(dtype, hipLaunchKernelGGL(embedding_kernel<DT>, dim3(rows), dim3(256), 0, as_stream(stream), ids, table,
                                      out, d, vocab));
  O355_CHECK_LAUNCH();
}

// Activation column gather for act-order int4 weights: out[m][k] = x[m][perm[k]] (16-bit elements).
namespace {
__global__ __launch_bounds__(256) void gather_columns_kernel(const uint16_t* __restrict__ x,
                                                             const int32_t* __restrict__ perm,
                                                             uint16_t* __restrict__ out, int K) {
  const uint16_t* xr = x + (int64_t)blockIdx.y * K;
  uint16_t* orow = out + (int64_t)blockIdx.y * K;
  const int k = (blockIdx.x * 256 + threadIdx.x) * 2;  // two outputs per thread: one 32-bit store
  if (k + 1 < K) {
    const uint32_t lo = xr[perm[k]], hi = xr[perm[k + 1]];
    *reinterpret_cast<uint32_t*>(orow + k) = lo | (hi << 16);
  } else if (k < K) {
    orow[k] = xr[perm[k]];
  }
}
}  // namespace

extern "C" int olmo355_gather_columns(const uint16_t* x, const int32_t* perm, uint16_t* out, int M, int K,
                                      void* stream) {
  if (!x || !perm || !out || M <= 0 || K <= 0) return O355_EINVAL;
  if (M > 65535 || (K & 1)) return O355_EUNSUPPORTED;
  hipLaunchKernelGGL(gather_columns_kernel, dim3((unsigned)((K / 2 + 255) / 256), (unsigned)M), dim3(256), 0,
                     as_stream(stream), x, perm, out, K);
  O355_CHECK_LAUNCH();
}

// x := min(max(x, -c), c) in place (clip_qkv)
namespace {
template <int DT>
__global__ __launch_bounds__(256) void clamp_kernel(void* __restrict__ x, int64_t n, float c) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) Act<DT>::st(x, i, fminf(fmaxf(Act<DT>::ld(x, i), -c), c));
}
}  // namespace

extern "C" int olmo355_clamp(void* x, int64_t n, float c, int dtype, void* stream) {
  if (!x || n <= 0 || !(c > 0.f)) return O355_EINVAL;
  DT_SWITCH(dtype, hipLaunchKernelGGL(clamp_kernel<DT>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream),
                                      x, n, c));
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_add(const void* a, const void* b, void* out, int64_t n, int dtype, void* stream) {
  if (!a || !b || !out || n <= 0) return O355_EINVAL;
  DT_SWITCH(dtype, hipLaunchKernelGGL(add_kernel<DT>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                                      as_stream(stream), a, b, out, n));
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_add_bias_bf16(const uint16_t* x, const uint16_t* bias_f16, uint16_t* out, int M, int N, void* stream) {
  if (!x || !bias_f16 || !out || M <= 0 || N <= 0) return O355_EINVAL;
  const int64_t total = (int64_t)M * N;
  hipLaunchKernelGGL(add_bias_bf16_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, as_stream(stream), x,
                     bias_f16, out, total, N);
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_add_bias_f16(const uint16_t* x, const uint16_t* bias_f16, uint16_t* out, int M, int N, void* stream) {
  if (!x || !bias_f16 || !out || M <= 0 || N <= 0) return O355_EINVAL;
  const int64_t total = (int64_t)M * N;
  hipLaunchKernelGGL(add_bias_f16_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, as_stream(stream), x,
                     bias_f16, out, total, N);
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_argmax(const void* logits, int64_t* out, int rows, int n, int dtype, void* stream) {
  if (!logits || !out || rows <= 0 || n <= 0) return O355_EINVAL;
  DT_SWITCH(dtype,
            hipLaunchKernelGGL(argmax_kernel<DT>, dim3(rows), dim3(1024), 0, as_stream(stream), logits, out, n));
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_greedy_next(const void* logits, int64_t* ids_out, const void* table, void* x_next, int rows, int n,
                                   int d, int vocab, int32_t* pos, const float* sin_tab, const float* cos_tab,
                                   float* rope_now, int hd, int n_pos, int dtype, void* stream) {
  if (!logits || !ids_out || !table || !x_next || !pos || !sin_tab || !cos_tab || !rope_now) return O355_EINVAL;
  if (rows <= 0 || n <= 0 || d <= 0 || vocab <= 0 || hd <= 0 || n_pos <= 0) return O355_EINVAL;
  DT_SWITCH(dtype, hipLaunchKernelGGL(greedy_next_kernel<DT>, dim3(rows), dim3(1024), 0, as_stream(stream), logits,
                                      ids_out, n, table, x_next, d, vocab, pos, sin_tab, cos_tab, rope_now, hd, n_pos));
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_incr_i32(int32_t* p, void* stream) {
  if (!p) return O355_EINVAL;
  hipLaunchKernelGGL(incr_kernel, dim3(1), dim3(1), 0, as_stream(stream), p);
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_version(void) { return 1; }

extern "C" const char* olmo355_status_string(int status) {
  switch (status) {
    case O355_OK: return "ok";
    case O355_EINVAL: return "invalid argument (null pointer or bad size)";
    case O355_EUNSUPPORTED: return "unsupported shape, dtype or group size";
    case O355_ELAUNCH: return "kernel launch failed";
    case O355_ETOOBIG: return "sizes exceed the fixed scratch of this entry point";
    default: return "unknown status";
  }
}
