// Bandwidth-bound row kernels: RMSNorm (+ residual add), non-parametric LayerNorm, QK-norm +
// rotary + KV-cache write, SwiGLU, embedding lookup, residual add, argmax.
// Rounding points follow the reference op by op so that a 16-bit activation dtype gives the
// same values as the reference's eager op chains.
#include "common.h"

namespace {

// ---- RMSNorm: olmo/model.py:241-255 ---------------------------------------------------------------
// fp32 normalise -> round to dtype -> multiply by weight in dtype (second rounding) -> optional
// residual add in dtype (third rounding).
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
template <int DT>
__global__ __launch_bounds__(256) void qknorm_rope_kernel(const void* __restrict__ qkv, const void* __restrict__ qw,
                                                          const void* __restrict__ kw, const float* __restrict__ sin_t,
                                                          const float* __restrict__ cos_t, void* __restrict__ q_out,
                                                          void* __restrict__ kc, void* __restrict__ vc, int T, int H,
                                                          int Hkv, int hd, int Lmax, int past_len,
                                                          const int32_t* __restrict__ past_dev, float eps) {
  __shared__ float red[16];
  const int row = blockIdx.x;  // b*T + t
  const int b = row / T, t = row % T;
  const int dq = H * hd, dk = Hkv * hd;
  const int64_t in_base = (int64_t)row * (dq + 2 * dk);
  const int past = past_dev ? *past_dev : past_len;
  const int pos = past + t;
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
  // q: pairs (j, j+half) inside each head
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

template <int DT>
__global__ __launch_bounds__(256) void embedding_kernel(const int64_t* __restrict__ ids, const void* __restrict__ tab,
                                                        void* __restrict__ out, int d, int vocab) {
  int64_t id = ids[blockIdx.x];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  typedef typename Act<DT>::T T;
  const T* src = (const T*)tab + id * d;
  T* dst = (T*)out + (int64_t)blockIdx.x * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) dst[i] = src[i];
}

template <int DT>
__global__ __launch_bounds__(256) void add_kernel(const void* __restrict__ a, const void* __restrict__ b,
                                                  void* __restrict__ out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) Act<DT>::st(out, i, Act<DT>::ld(a, i) + Act<DT>::ld(b, i));
}

// first index of the maximum of each row (torch.argmax tie rule)
template <int DT>
__global__ __launch_bounds__(1024) void argmax_kernel(const void* __restrict__ x, int64_t* __restrict__ out, int n) {
  __shared__ float sv[16];
  __shared__ int si[16];
  const int64_t base = (int64_t)blockIdx.x * n;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = Act<DT>::ld(x, base + i);
    if (v > best || (v == best && i < bi)) best = v, bi = i;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (ov > best || (ov == best && oi < bi)) best = ov, bi = oi;
  }
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) sv[w] = best, si[w] = bi;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i)
      if (sv[i] > best || (sv[i] == best && si[i] < bi)) best = sv[i], bi = si[i];
    out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
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
  } else {                                                  \
    return O355_EUNSUPPORTED;                               \
  }

extern "C" int olmo355_rmsnorm(const void* x, const void* weight, const void* residual, void* out, int rows, int d,
                               float eps, int dtype, void* stream) {
  if (!x || !out || rows <= 0 || d <= 0) return O355_EINVAL;
  DT_SWITCH(dtype, hipLaunchKernelGGL(rmsnorm_kernel<DT>, dim3(rows), dim3(256), 0, as_stream(stream), x, weight,
                                      residual, out, d, eps));
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
  DT_SWITCH(dtype, hipLaunchKernelGGL(qknorm_rope_kernel<DT>, dim3(B * T), dim3(256), 0, as_stream(stream), qkv, qw, kw,
                                      sin_tab, cos_tab, q_out, kcache, vcache, T, H, Hkv, hd, Lmax, past_len,
                                      past_len_dev, eps));
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_swiglu(const void* x, void* out, int rows, int h, int dtype, void* stream) {
  if (!x || !out || rows <= 0 || h <= 0) return O355_EINVAL;
  const int64_t total = (int64_t)rows * h;
  DT_SWITCH(dtype, hipLaunchKernelGGL(swiglu_kernel<DT>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                                      as_stream(stream), x, out, total, h));
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_embedding(const int64_t* ids, const void* table, void* out, int rows, int d, int vocab,
                                 int dtype, void* stream) {
  if (!ids || !table || !out || rows <= 0 || d <= 0 || vocab <= 0) return O355_EINVAL;
  DT_SWITCH(dtype, hipLaunchKernelGGL(embedding_kernel<DT>, dim3(rows), dim3(256), 0, as_stream(stream), ids, table,
                                      out, d, vocab));
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_add(const void* a, const void* b, void* out, int64_t n, int dtype, void* stream) {
  if (!a || !b || !out || n <= 0) return O355_EINVAL;
  DT_SWITCH(dtype, hipLaunchKernelGGL(add_kernel<DT>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                                      as_stream(stream), a, b, out, n));
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_argmax(const void* logits, int64_t* out, int rows, int n, int dtype, void* stream) {
  if (!logits || !out || rows <= 0 || n <= 0) return O355_EINVAL;
  DT_SWITCH(dtype,
            hipLaunchKernelGGL(argmax_kernel<DT>, dim3(rows), dim3(1024), 0, as_stream(stream), logits, out, n));
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
    default: return "unknown status";
  }
}
