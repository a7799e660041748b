// Causal attention over the contiguous per-layer KV cache [B, Hkv, Lmax, hd]
// (olmo/model.py:533-586,627-648): softmax(q k^T / sqrt(hd) + bias) v, fp32 softmax.
//
//  * attn_prefill_mfma_kernel  bf16, hd 64/128: flash-style, K and V^T tiles staged in LDS in
//    MFMA-fragment order, S^T = K.Q^T and O^T = V^T.P^T on the matrix cores so the softmax
//    statistics of a query stay in one lane column and P never leaves registers.
//  * attn_decode_kernel        one query per sequence, keys split over workgroups and waves,
//    DPP / wave reductions, partial (max, sum, o) merged by attn_decode_combine_kernel.
//  * attn_generic_kernel       any dtype / head size <= 128, one query per thread (used for the
//    fp32 model configuration).
//
// Masking: keys after the query position are skipped.  A key whose key_bias entry is <= -1e30
// (padding) keeps a *finite* score, the dtype's most negative value, as in the reference
// (olmo/model.py:1337-1376, olmo/torch_util.py:81-90): a query that sees only padding gets the
// plain average of the values it sees instead of NaN.
#include "common.h"

namespace {

constexpr float kMaskThreshold = -1e30f;

// 8 consecutive channels as floats: one 16-byte vector of bf16 or two of fp32
template <int DT> struct Vec8;
template <> struct Vec8<O355_BF16> {
  static __device__ __forceinline__ void unpack(const u32x4 (&r)[1], float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[2 * i] = bf16lo_to_f32(r[0][i]), f[2 * i + 1] = bf16hi_to_f32(r[0][i]);
  }
  static __device__ __forceinline__ void ld(const void* p, int64_t elem, float (&f)[8]) {
    u32x4 r[1] = {reinterpret_cast<const u32x4*>(p)[elem >> 3]};
    unpack(r, f);
  }
};
template <> struct Vec8<O355_F32> {
  static __device__ __forceinline__ void unpack(const u32x4 (&r)[2], float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(r[0][i]), f[4 + i] = __uint_as_float(r[1][i]);
  }
  static __device__ __forceinline__ void ld(const void* p, int64_t elem, float (&f)[8]) {
    u32x4 r[2] = {reinterpret_cast<const u32x4*>(p)[elem >> 2], reinterpret_cast<const u32x4*>(p)[(elem >> 2) + 1]};
    unpack(r, f);
  }
};

// =====================================================================================================
// generic: one thread per query row, K/V tiles of 32 keys in LDS as fp32
// =====================================================================================================
template <int DT, int HD>
__global__ __launch_bounds__(64) void attn_generic_kernel(const void* __restrict__ q, const void* __restrict__ kc,
                                                          const void* __restrict__ vc,
                                                          const float* __restrict__ key_bias, void* __restrict__ out,
                                                          int T, int H, int Hkv, int Lmax, int past_len,
                                                          int bias_stride) {
  constexpr int KT = 32;
  __shared__ float sk[KT][HD + 1], sv[KT][HD + 1], sb[KT];
  const int b = blockIdx.z, h = blockIdx.y, hk = h / (H / Hkv);
  const int t = blockIdx.x * 64 + threadIdx.x;
  const int tq = t < T ? t : T - 1;
  const int pos = past_len + tq;
  const int last_pos = past_len + min(blockIdx.x * 64 + 63, T - 1);
  const float scale = 1.f / sqrtf((float)HD);
  const float lowest = Act<DT>::lowest();
  float qr[HD], acc[HD];
  const int64_t qbase = ((int64_t)b * T + tq) * H * HD + (int64_t)h * HD;
#pragma unroll
  for (int i = 0; i < HD; ++i) qr[i] = Act<DT>::ld(q, qbase + i), acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  const int64_t cbase = ((int64_t)b * Hkv + hk) * Lmax * HD;
  for (int k0 = 0; k0 <= last_pos; k0 += KT) {
    __syncthreads();
    for (int e = threadIdx.x; e < KT * HD; e += 64) {
      const int kk = e / HD, i = e % HD;
      const int key = min(k0 + kk, last_pos);
      sk[kk][i] = Act<DT>::ld(kc, cbase + (int64_t)key * HD + i);
      sv[kk][i] = Act<DT>::ld(vc, cbase + (int64_t)key * HD + i);
    }
    if (threadIdx.x < KT) {
      const int key = min(k0 + (int)threadIdx.x, last_pos);
      sb[threadIdx.x] = key_bias ? key_bias[(int64_t)b * bias_stride + key] : 0.f;
    }
    __syncthreads();
    const int kend = min(KT, pos - k0 + 1);
    for (int kk = 0; kk < kend; ++kk) {
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < HD; ++i) s = __builtin_fmaf(qr[i], sk[kk][i], s);
      s = sb[kk] <= kMaskThreshold ? lowest : s * scale + sb[kk];
      const float mn = fmaxf(m, s);
      const float alpha = expf(m - mn), p = expf(s - mn);
      l = l * alpha + p;
#pragma unroll
      for (int i = 0; i < HD; ++i) acc[i] = acc[i] * alpha + p * sv[kk][i];
      m = mn;
    }
  }
  if (t < T) {
    const float inv = 1.f / l;
#pragma unroll
    for (int i = 0; i < HD; ++i) Act<DT>::st(out, qbase + i, acc[i] * inv);
  }
}

// =====================================================================================================
// prefill on the matrix cores (bf16)
// =====================================================================================================
// Workgroup: 4 waves x 32 queries = 128 queries of one (batch, head); KV tile: 64 keys.
// LDS  K  : [key-tile 4][hd-step HD/32][64 lanes][8 bf16]   A operand of S^T = K . Q^T
//      V^T: [hd-tile HD/16][key-step 2][64 lanes][8 bf16]   A operand of O^T = V^T . P^T
// In the second product the 8 key slots of lane group kq in key-step s are
//   e<4 : key 32s + 4kq + e        e>=4 : key 32s + 16 + 4kq + (e-4)
// which is exactly how the S^T accumulators of the two 16-key tiles 2s, 2s+1 sit in a lane, so
// P goes from accumulator registers to the B operand without leaving the lane.
template <int HD>
__global__ __launch_bounds__(256) void attn_prefill_mfma_kernel(const uint16_t* __restrict__ q,
                                                                const uint16_t* __restrict__ kc,
                                                                const uint16_t* __restrict__ vc,
                                                                const float* __restrict__ key_bias,
                                                                uint16_t* __restrict__ out, int T, int H, int Hkv,
                                                                int Lmax, int past_len, int bias_stride) {
  constexpr int KT = 64;             // keys per tile
  constexpr int STEPS = HD / 32;     // hd steps of the first product
  constexpr int HT = HD / 16;        // hd tiles of the second product
  constexpr int QT = 2;              // 16-query tiles per wave
  __shared__ __align__(16) u32x4 lds_k[4 * STEPS * 64];
  __shared__ __align__(16) u32x4 lds_v[HT * 2 * 64];
  __shared__ float lds_bias[KT];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, kq = lane >> 4;
  // heavier (later) query blocks first: they have the most key tiles
  const int qblock = gridDim.x - 1 - blockIdx.x;
  const int b = blockIdx.z, h = blockIdx.y, hk = h / (H / Hkv);
  const int q0 = qblock * 128 + wave * 32;
  const float scale = 1.f / sqrtf((float)HD);
  const float lowest = -3.3895313892515355e38f;
  const int64_t cbase = ((int64_t)b * Hkv + hk) * Lmax * HD;

  // Q^T fragments: lane (query col, hd 32*step + 8*kq ..)
  bf16x8 qf[QT][STEPS];
  int qpos[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int t = min(q0 + qt * 16 + col, T - 1);
    qpos[qt] = past_len + t;
    const uint16_t* src = q + ((int64_t)b * T + t) * H * HD + (int64_t)h * HD;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) qf[qt][s] = *reinterpret_cast<const bf16x8*>(src + 32 * s + 8 * kq);
  }
  f32x4 o[QT][HT];
  float m[QT], l[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    m[qt] = -INFINITY, l[qt] = 0.f;
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) o[qt][ht] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int last_pos = past_len + min(qblock * 128 + 127, T - 1);   // workgroup-uniform loop bound
  const int wave_last = past_len + min(q0 + 31, T - 1);             // last position this wave needs
  for (int k0 = 0; k0 <= last_pos; k0 += KT) {
    __syncthreads();
    // ---- stage K: 64 keys x HD, 16-byte chunks ------------------------------------------------------
    constexpr int CPR = HD / 8;  // chunks per key row
    for (int e = tid; e < KT * CPR; e += 256) {
      const int kk = e / CPR, c = e % CPR;
      const int key = min(k0 + kk, last_pos);
      const u32x4 v = *reinterpret_cast<const u32x4*>(kc + cbase + (int64_t)key * HD + 8 * c);
      lds_k[((kk >> 4) * STEPS + (c >> 2)) * 64 + (kk & 15) + 16 * (c & 3)] = v;
    }
    // ---- stage V^T: key pairs (kk, kk+1) x 8 hd values -> 8 dword writes -------------------------------
    for (int e = tid; e < (KT / 2) * CPR; e += 256) {
      const int kp = e / CPR, c = e % CPR;
      const int kk = 2 * kp;
      const int key0 = min(k0 + kk, last_pos), key1 = min(k0 + kk + 1, last_pos);
      const u32x4 v0 = *reinterpret_cast<const u32x4*>(vc + cbase + (int64_t)key0 * HD + 8 * c);
      const u32x4 v1 = *reinterpret_cast<const u32x4*>(vc + cbase + (int64_t)key1 * HD + 8 * c);
      const int kt = kk >> 4, s2 = kt >> 1, hf = kt & 1, k16 = kk & 15;
      const int kq_ = k16 >> 2, e0 = (k16 & 3) + 4 * hf;  // e0 even
      uint32_t* dst = reinterpret_cast<uint32_t*>(lds_v);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int hd_ = 8 * c + i;
        const int ht = hd_ >> 4, lo = hd_ & 15;
        const uint32_t a = (i & 1) ? (v0[i >> 1] >> 16) : (v0[i >> 1] & 0xffffu);
        const uint32_t bb = (i & 1) ? (v1[i >> 1] >> 16) : (v1[i >> 1] & 0xffffu);
        dst[(((ht * 2 + s2) * 64 + kq_ * 16 + lo) * 8 + e0) >> 1] = a | (bb << 16);
      }
    }
    if (tid < KT) {
      const int key = min(k0 + tid, last_pos);
      lds_bias[tid] = key_bias ? key_bias[(int64_t)b * bias_stride + key] : 0.f;
    }
    __syncthreads();
    if (k0 > wave_last) continue;  // nothing visible to this wave in the tile (barriers stay uniform)

    // ---- S^T = K . Q^T -----------------------------------------------------------------------------
    f32x4 s[QT][4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) s[qt][kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int st = 0; st < STEPS; ++st) {
        const bf16x8 kf = __builtin_bit_cast(bf16x8, lds_k[(kt * STEPS + st) * 64 + lane]);
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) s[qt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[qt][st], s[qt][kt], 0, 0, 0);
      }
    }
    // ---- online softmax per query column ----------------------------------------------------------------
    bf16x8 pf[QT][2];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      float tmax = -INFINITY;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int kk = kt * 16 + 4 * kq + r;
          const int key = k0 + kk;
          const float bias = lds_bias[kk];
          float v = bias <= kMaskThreshold ? lowest : s[qt][kt][r] * scale + bias;
          v = key > qpos[qt] ? -INFINITY : v;
          s[qt][kt][r] = v;
          tmax = fmaxf(tmax, v);
        }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float mn = fmaxf(m[qt], tmax);  // finite: key 0 of the first tile is visible to every query
      const float alpha = __expf(m[qt] - mn);
      float psum = 0.f;
      float p[4][4];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          p[kt][r] = __expf(s[qt][kt][r] - mn);
          psum += p[kt][r];
        }
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
      l[qt] = l[qt] * alpha + psum;
      m[qt] = mn;
#pragma unroll
      for (int ht = 0; ht < HT; ++ht)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[qt][ht][r] *= alpha;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        u32x4 w;
        w.x = pack_bf16x2(p[2 * s2][0], p[2 * s2][1]);
        w.y = pack_bf16x2(p[2 * s2][2], p[2 * s2][3]);
        w.z = pack_bf16x2(p[2 * s2 + 1][0], p[2 * s2 + 1][1]);
        w.w = pack_bf16x2(p[2 * s2 + 1][2], p[2 * s2 + 1][3]);
        pf[qt][s2] = __builtin_bit_cast(bf16x8, w);
      }
    }
    // ---- O^T += V^T . P^T ----------------------------------------------------------------------------------
#pragma unroll
    for (int ht = 0; ht < HT; ++ht)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const bf16x8 vf = __builtin_bit_cast(bf16x8, lds_v[(ht * 2 + s2) * 64 + lane]);
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) o[qt][ht] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[qt][s2], o[qt][ht], 0, 0, 0);
      }
  }
  // ---- write O[q][hd]: lane holds hd = 16ht + 4kq + r for query col ------------------------------------------
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int t = q0 + qt * 16 + col;
    if (t >= T) continue;
    const float inv = 1.f / l[qt];
    uint16_t* dst = out + ((int64_t)b * T + t) * H * HD + (int64_t)h * HD;
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) {
      u32x2 w;
      w.x = pack_bf16x2(o[qt][ht][0] * inv, o[qt][ht][1] * inv);
      w.y = pack_bf16x2(o[qt][ht][2] * inv, o[qt][ht][3] * inv);
      *reinterpret_cast<u32x2*>(dst + 16 * ht + 4 * kq) = w;
    }
  }
}

// =====================================================================================================
// decode: one query per (batch, head); keys split into chunks of 128 (32 per wave)
// =====================================================================================================
// A lane owns 8 channels of one key: LPK = HD/8 lanes cover a key row with one 16-byte load each,
// a wave covers 64/LPK keys per load instruction.  All K and V loads of the wave's 32 keys are
// issued before the first use (the kernel is latency-bound at batch 1); the dot product is reduced
// over the LPK lanes with DPP adds.
constexpr int kDecodeChunk = 128;
constexpr int kDecodeKeysPerWave = 32;

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
  return v + __builtin_bit_cast(float, t);
}
// sum over aligned groups of W lanes (W = 4, 8 or 16); every lane of the group gets the sum
template <int W>
__device__ __forceinline__ float group_sum(float v) {
  v = dpp_add<0xB1>(v);                          // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);                          // quad_perm [2,3,0,1]
  if constexpr (W >= 8) v = dpp_add<0x141>(v);   // row_half_mirror
  if constexpr (W >= 16) v = dpp_add<0x140>(v);  // row_mirror
  return v;
}

template <int DT, int HD>
__global__ __launch_bounds__(256) void attn_decode_kernel(const void* __restrict__ q, const void* __restrict__ kc,
                                                          const void* __restrict__ vc,
                                                          const float* __restrict__ key_bias, float* __restrict__ ws,
                                                          int H, int Hkv, int Lmax, int past_len,
                                                          const int32_t* __restrict__ past_dev, int nchunks_max,
                                                          int bias_stride) {
  constexpr int LPK = HD / 8;                        // lanes per key (8 channels each)
  constexpr int KPI = 64 / LPK;                      // keys per wave iteration
  constexpr int ITERS = kDecodeKeysPerWave / KPI;    // iterations per wave
  constexpr int VW = DT == O355_BF16 ? 1 : 2;        // 16-byte vectors per 8 channels
  __shared__ float red_o[4][HD];
  __shared__ float red_ml[4][2];
  const int chunk = blockIdx.x, h = blockIdx.y, b = blockIdx.z, hk = h / (H / Hkv);
  const int L = (past_dev ? *past_dev : past_len) + 1;
  if (chunk * kDecodeChunk >= L) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = lane % LPK, kslot = lane / LPK;
  const float scale = 1.f / sqrtf((float)HD);
  const float lowest = Act<DT>::lowest();
  const int64_t cbase = ((int64_t)b * Hkv + hk) * Lmax * HD;
  const int kbase = chunk * kDecodeChunk + wave * kDecodeKeysPerWave;

  // ---- every load of this wave, issued up front -------------------------------------------------
  u32x4 kreg[ITERS][VW], vreg[ITERS][VW];
  float bias[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int keyc = min(kbase + it * KPI + kslot, L - 1);
    const int64_t e = cbase + (int64_t)keyc * HD + sub * 8;
#pragma unroll
    for (int v = 0; v < VW; ++v) kreg[it][v] = reinterpret_cast<const u32x4*>(kc)[e * VW / 8 + v];
  }
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int keyc = min(kbase + it * KPI + kslot, L - 1);
    const int64_t e = cbase + (int64_t)keyc * HD + sub * 8;
#pragma unroll
    for (int v = 0; v < VW; ++v) vreg[it][v] = reinterpret_cast<const u32x4*>(vc)[e * VW / 8 + v];
    bias[it] = key_bias ? key_bias[(int64_t)b * bias_stride + keyc] : 0.f;
  }
  float qr[8];
  Vec8<DT>::ld(q, ((int64_t)b * H + h) * HD + sub * 8, qr);

  float s[ITERS];
  float wmax = -INFINITY;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int key = kbase + it * KPI + kslot;
    float kf[8];
    Vec8<DT>::unpack(kreg[it], kf);
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) d = __builtin_fmaf(qr[i], kf[i], d);
    d = group_sum<LPK>(d);
    float v = bias[it] <= kMaskThreshold ? lowest : d * scale + bias[it];
    v = key < L ? v : -INFINITY;
    s[it] = v;
    wmax = fmaxf(wmax, v);
  }
#pragma unroll
  for (int o = LPK; o < 64; o <<= 1) wmax = fmaxf(wmax, __shfl_xor(wmax, o, 64));
  // a wave whose keys all lie beyond L contributes nothing
  const bool empty = (kbase >= L);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float lsum = 0.f;
  if (!empty) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const float p = __expf(s[it] - wmax);  // exp(-inf) = 0 for keys beyond L
      lsum += p;
      float vf[8];
      Vec8<DT>::unpack(vreg[it], vf);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(p, vf[i], acc[i]);
    }
    // sum over the key slots of the wave (lanes with equal `sub`)
#pragma unroll
    for (int o = LPK; o < 64; o <<= 1) {
      lsum += __shfl_xor(lsum, o, 64);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += __shfl_xor(acc[i], o, 64);
    }
  }
  if (lane < LPK) {
#pragma unroll
    for (int i = 0; i < 8; ++i) red_o[wave][sub * 8 + i] = acc[i];
  }
  if (lane == 0) red_ml[wave][0] = empty ? -INFINITY : wmax, red_ml[wave][1] = empty ? 0.f : lsum;
  __syncthreads();
  // merge the 4 waves; wave 0 always has at least one key
  float mm = red_ml[0][0];
#pragma unroll
  for (int w = 1; w < 4; ++w) mm = fmaxf(mm, red_ml[w][0]);
  float* dst = ws + (((int64_t)b * H + h) * nchunks_max + chunk) * (HD + 2);
  if (tid < HD) {
    float ov = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) ov += red_o[w][tid] * __expf(red_ml[w][0] - mm);
    dst[tid] = ov;
  }
  if (tid == 0) {
    float lv = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) lv += red_ml[w][1] * __expf(red_ml[w][0] - mm);
    dst[HD] = mm;
    dst[HD + 1] = lv;
  }
}

template <int DT, int HD>
__global__ __launch_bounds__(HD) void attn_decode_combine_kernel(const float* __restrict__ ws, void* __restrict__ out,
                                                                 int H, int past_len,
                                                                 const int32_t* __restrict__ past_dev,
                                                                 int nchunks_max) {
  constexpr int UN = 8;  // partials fetched per round, all loads before the first use
  const int h = blockIdx.x, b = blockIdx.y;
  const int L = (past_dev ? *past_dev : past_len) + 1;
  const int nch = (L + kDecodeChunk - 1) / kDecodeChunk;
  const float* src = ws + ((int64_t)b * H + h) * nchunks_max * (HD + 2);
  float mm = -INFINITY, ov = 0.f, lv = 0.f;
  for (int c0 = 0; c0 < nch; c0 += UN) {
    float m[UN], l[UN], o[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int c = min(c0 + u, nch - 1);
      m[u] = src[c * (HD + 2) + HD], l[u] = src[c * (HD + 2) + HD + 1], o[u] = src[c * (HD + 2) + threadIdx.x];
    }
    float rm = mm;
#pragma unroll
    for (int u = 0; u < UN; ++u)
      if (c0 + u < nch) rm = fmaxf(rm, m[u]);
    const float a = __expf(mm - rm);  // exp(-inf) = 0 on the first round
    ov *= a, lv *= a;
#pragma unroll
    for (int u = 0; u < UN; ++u)
      if (c0 + u < nch) {
        const float w = __expf(m[u] - rm);
        ov += o[u] * w, lv += l[u] * w;
      }
    mm = rm;
  }
  Act<DT>::st(out, ((int64_t)b * H + h) * HD + threadIdx.x, ov / lv);
}

template <int DT, int HD>
int launch_decode(const void* q, const void* kc, const void* vc, const float* key_bias, void* out, float* ws, int B,
                  int H, int Hkv, int Lmax, int past_len, const int32_t* past_dev, int n_keys_max, int bias_stride,
                  hipStream_t stream) {
  const int nch = (n_keys_max + kDecodeChunk - 1) / kDecodeChunk;
  hipLaunchKernelGGL((attn_decode_kernel<DT, HD>), dim3(nch, H, B), dim3(256), 0, stream, q, kc, vc, key_bias, ws, H,
                     Hkv, Lmax, past_len, past_dev, nch, bias_stride);
  hipLaunchKernelGGL((attn_decode_combine_kernel<DT, HD>), dim3(H, B), dim3(HD), 0, stream, ws, out, H, past_len,
                     past_dev, nch);
  O355_CHECK_LAUNCH();
}

template <int DT, int HD>
int launch_generic(const void* q, const void* kc, const void* vc, const float* key_bias, void* out, int B, int T, int H,
                   int Hkv, int Lmax, int past_len, int bias_stride, hipStream_t stream) {
  hipLaunchKernelGGL((attn_generic_kernel<DT, HD>), dim3((T + 63) / 64, H, B), dim3(64), 0, stream, q, kc, vc, key_bias,
                     out, T, H, Hkv, Lmax, past_len, bias_stride);
  O355_CHECK_LAUNCH();
}

}  // namespace

extern "C" int olmo355_attn_prefill(const void* q, const void* kcache, const void* vcache, const float* key_bias,
                                    void* out, int B, int T, int H, int Hkv, int hd, int Lmax, int past_len,
                                    int bias_stride, int dtype, void* stream) {
  if (!q || !kcache || !vcache || !out) return O355_EINVAL;
  if (B <= 0 || T <= 0 || H <= 0 || Hkv <= 0 || H % Hkv || past_len < 0 || past_len + T > Lmax) return O355_EINVAL;
  if (key_bias && bias_stride < past_len + T) return O355_EINVAL;
  hipStream_t s = as_stream(stream);
  if (dtype == O355_BF16 && (hd == 128 || hd == 64)) {
    const dim3 grid((T + 127) / 128, H, B);
    if (hd == 128)
      hipLaunchKernelGGL(attn_prefill_mfma_kernel<128>, grid, dim3(256), 0, s, (const uint16_t*)q,
                         (const uint16_t*)kcache, (const uint16_t*)vcache, key_bias, (uint16_t*)out, T, H, Hkv, Lmax,
                         past_len, bias_stride);
    else
      hipLaunchKernelGGL(attn_prefill_mfma_kernel<64>, grid, dim3(256), 0, s, (const uint16_t*)q,
                         (const uint16_t*)kcache, (const uint16_t*)vcache, key_bias, (uint16_t*)out, T, H, Hkv, Lmax,
                         past_len, bias_stride);
    O355_CHECK_LAUNCH();
  }
#define GENERIC(DTv, HDv) \
  return launch_generic<DTv, HDv>(q, kcache, vcache, key_bias, out, B, T, H, Hkv, Lmax, past_len, bias_stride, s)
  if (dtype == O355_F32) {
    if (hd == 32) GENERIC(O355_F32, 32);
    if (hd == 64) GENERIC(O355_F32, 64);
    if (hd == 128) GENERIC(O355_F32, 128);
  } else if (dtype == O355_BF16) {
    if (hd == 32) GENERIC(O355_BF16, 32);
  }
#undef GENERIC
  return O355_EUNSUPPORTED;
}

extern "C" int64_t olmo355_attn_decode_workspace_bytes(int B, int H, int hd, int n_keys_max) {
  if (B <= 0 || H <= 0 || hd <= 0 || n_keys_max <= 0) return 0;
  const int64_t nch = (n_keys_max + kDecodeChunk - 1) / kDecodeChunk;
  return (int64_t)B * H * nch * (hd + 2) * 4;
}

extern "C" int olmo355_attn_decode(const void* q, const void* kcache, const void* vcache, const float* key_bias,
                                   void* out, void* ws, int B, int H, int Hkv, int hd, int Lmax, int past_len,
                                   const int32_t* past_len_dev, int n_keys_max, int bias_stride, int dtype,
                                   void* stream) {
  if (!q || !kcache || !vcache || !out || !ws) return O355_EINVAL;
  if (B <= 0 || H <= 0 || Hkv <= 0 || H % Hkv || past_len < 0 || n_keys_max <= 0 || n_keys_max > Lmax)
    return O355_EINVAL;
  if (!past_len_dev && past_len + 1 > n_keys_max) return O355_EINVAL;
  if (key_bias && bias_stride < n_keys_max) return O355_EINVAL;
  hipStream_t s = as_stream(stream);
#define DECODE(DTv, HDv)                                                                                          \
  return launch_decode<DTv, HDv>(q, kcache, vcache, key_bias, out, (float*)ws, B, H, Hkv, Lmax, past_len, \
                                 past_len_dev, n_keys_max, bias_stride, s)
  if (dtype == O355_BF16) {
    if (hd == 128) DECODE(O355_BF16, 128);
    if (hd == 64) DECODE(O355_BF16, 64);
    if (hd == 32) DECODE(O355_BF16, 32);
  } else if (dtype == O355_F32) {
    if (hd == 128) DECODE(O355_F32, 128);
    if (hd == 64) DECODE(O355_F32, 64);
    if (hd == 32) DECODE(O355_F32, 32);
  }
#undef DECODE
  return O355_EUNSUPPORTED;
}
