// The batch-1 decode step as a relay of launches on two streams.
//
// A decode step is a chain of short bandwidth-bound launches (att_proj -> attention -> attn_out -> ff_proj ->
// ff_out per block, olmo/model.py:746-823), each of which needs the whole output of the one before.  On one
// stream a launch of 9..47 MB spends about 4 us of its 5..12 us outside streaming: the boundary behind its
// predecessor, the latency of its first weight requests, the reduction tail.  Weights do not depend on
// activations, so here launch n+1 starts on a second stream as soon as launch n-1 has ended, requests ALL of its
// weights at once, and only then waits for the rows of launch n -- the next launch's stream fills the time in
// which this one finishes.
//
// The hand-over needs no flag, counter or ticket: every number that crosses from one launch to the next carries
// the step's epoch.  An output element is one 32-bit word (bf16 bits << 16 | epoch & 0xffff), a per-tile sum of
// squares one 32-bit word too (the float rounded to 20 mantissa bits | epoch & 0xf), each written with one
// device-scope store.  A consumer loads its
// slice of the row with device-coherent loads and looks at the tags: all equal to the epoch -> the numbers are
// this step's; otherwise it asks again.  Every buffer is written exactly once per step and the epoch changes with
// every step, so a stale word can never pass for a fresh one.  The wait is bounded: after `spin_limit` polls the
// wave sets `*status`, takes what it has and goes on, so every launch ends whatever happens around it.
//
// Two launches that wait on each other's streams must be able to live on the chip together: a younger launch whose
// waiting workgroups fill every CU would keep the older one's remaining workgroups from starting.  The host checks
// that before it uses the second stream (olmo355_relay_pair_ok): with n workgroups of the younger launch on a CU, one
// more of the older one must still fit (wave slots, registers, LDS) for every n the younger grid can put on all
// CUs at once.
//
// The kernels: w4_relay_kernel, the int4 linear at one row with the "four groups share one MFMA accumulator"
// scheme of w4_gemv_small_kernel (gemv.hip), every weight piece of a wave requested before the wait; prologue
// x := resid + rmsnorm(a) from the producer's per-tile sums of squares (olmo/model.py:241-255,786-794), epilogues
// SwiGLU (olmo/model.py:365-368) and per-tile sums of squares; relay_final_kernel, the last block's pending
// residual update from tagged inputs into a plain bf16 row.  The attention launch of the relay is
// attn_decode_fused_kernel<.., RELAY = true> (attention.hip).
#include <algorithm>
#include <type_traits>

#include "common.h"
#include "../../include/olmo355_debug.h"

namespace {

constexpr int kSc1 = 16;  // cache policy of a buffer access: device-coherent (never served from a stale L2 line)
constexpr int kHintCopies = O355_RELAY_HINT_COPIES, kHintStride = O355_RELAY_HINT_STRIDE;

struct RelayArgs {
  const void* x;           // [K]: tagged words (x_tagged) or plain bf16
  const uint32_t* ssq_in;  // norm: [K/16] tagged sums (float, low 4 bits = epoch & 0xf) left by the launch that wrote x
  const uint32_t* resid;   // norm: [K] tagged residual stream
  const uint16_t* norm_w;  // norm: [K] bf16
  uint32_t* x_out;         // norm: [K] tagged, resid + rmsnorm(x), written by workgroup 0
  void* y;                 // [N] (SwiGLU: [N/2]): tagged words (y_tagged) or plain bf16
  uint32_t* ssq_out;       // optional, [N/16] tagged sums
  const int32_t* epoch;    // the step's epoch (device word)
  int32_t* status;         // [0] set to 1 when a wait gave up; [1..3] statistics when [4] is set (8 words)
  const int32_t* hint_in;  // optional: a word the producer sets to the epoch when its last workgroup is done
  int32_t* hint_out;       // optional: this launch's own such word
  float eps;
  int N, K, x_tagged, y_tagged, spin_limit;
};

// At the top of every polling loop: the requests below it must be made again in every iteration.  (A buffer load is a
// plain read to the compiler; without this it may keep the first answer in a register and the loop never ends.)
__device__ __forceinline__ void poll_fence() { asm volatile("" ::: "memory"); }

__device__ __forceinline__ uint32_t tag_word(float v, uint32_t tag16) { return ((uint32_t)f32_to_bf16_bits(v) << 16) | tag16; }
// a sum of squares as a tagged word: rounded to 20 mantissa bits (its error then stays below that of adding the
// 256 .. 512 partials of a row in another order), the low 4 bits carry the epoch -- enough to tell this step's
// word from the previous step's, which is the only other thing the buffer can hold
__device__ __forceinline__ uint32_t tag_sum(float v, uint32_t epoch) { return ((__float_as_uint(v) + 0x8u) & 0xfffffff0u) | (epoch & 0xfu); }
__device__ __forceinline__ float sum_of(uint32_t w) { return __uint_as_float(w & 0xfffffff0u); }
__device__ __forceinline__ bool sums_ok(const u32x4& v, uint32_t epoch) {
  const uint32_t t = epoch & 0xfu;
  return (((v.x ^ t) | (v.y ^ t) | (v.z ^ t) | (v.w ^ t)) & 0xfu) == 0u;
}
__device__ __forceinline__ bool tags_ok(const u32x4& v, uint32_t tag16) {
  return (((v.x ^ tag16) | (v.y ^ tag16) | (v.z ^ tag16) | (v.w ^ tag16)) & 0xffffu) == 0u;
}
// four tagged words -> four bf16 in two words
__device__ __forceinline__ u32x2 untag4(const u32x4& v) {
  return u32x2{(v.x >> 16) | (v.y & 0xffff0000u), (v.z >> 16) | (v.w & 0xffff0000u)};
}

// MODE 0: plain bf16 activations; 1: tagged activations; 2: tagged activations with the chained-norm prologue.
// NQ: quads of four 128-row groups a wave holds in registers (its whole share of K: ceil(K/128 / WAVES) <= 4 NQ).
// Registers decide how many launches fit the chip side by side: the two-tile shapes are held to 96 (five waves per
// SIMD), the others are left to the compiler.
constexpr int relay_min_waves_per_simd(int NT, int NQ) { return 1; }

template <int NT, int WAVES, int NQ, int MODE, int EPI>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(relay_min_waves_per_simd(NT, NQ))))
void w4_relay_kernel(RelayArgs a, const u32x4* __restrict__ wt,
                                                              const uint16_t* __restrict__ st, const uint8_t* __restrict__ zt) {
  static_assert(EPI == 0 || NT == 2, "the SwiGLU epilogue owns one up tile and one gate tile");
  constexpr int XC = 2 * NQ;  // 256-element chunks of a wave's slice, at most
  extern __shared__ __align__(16) unsigned char smem[];
  const int K = a.K, G = K >> 7, ntiles = a.N >> 4;
  const int xbytes = K * 2;                                // LDS: the row, a zero row, the reduction area
  float* red = reinterpret_cast<float*>(smem + 2 * xbytes);  // [WAVES][NT][16]
  const uint16_t* xl = reinterpret_cast<const uint16_t*>(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int g_begin = (G * wave) / WAVES, g_end = (G * (wave + 1)) / WAVES;
  int tile[NT], tg[NT];
  if constexpr (EPI == 1) {
    tile[0] = blockIdx.x, tile[1] = blockIdx.x + (ntiles >> 1);
  } else {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) tile[nt] = blockIdx.x * NT + nt;
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) tg[nt] = min(tile[nt], ntiles - 1) * G;  // out-of-range tiles: computed, dropped

  // ---- 1. every weight piece of this wave, its scales and zeros: nothing here depends on another launch -----------
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(wt, (int64_t)ntiles * G * 1024);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(st, (int64_t)ntiles * G * 32);
  const __amdgpu_buffer_rsrc_t rz = make_rsrc(zt, (int64_t)ntiles * G * 8);
  u32x4 w[NQ][4][NT];
  uint32_t s16[NQ][NT], z8[NQ][NT];
  auto issue_weights = [&]() {
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int gc = min(g_begin + 4 * q + u, G - 1);  // past the wave's share: any valid piece, never multiplied
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          w[q][u][nt] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, lane * 16, (tg[nt] + gc) * 1024, 2));
      }
    // the lanes of row block kq hold the scale and zero of group 4 q + kq of the quad
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        s16[q][nt] = __builtin_amdgcn_raw_buffer_load_b16(rs, (kq * 16 + col) * 2, (tg[nt] + g_begin + 4 * q) * 32, 0);
        z8[q][nt] = __builtin_amdgcn_raw_buffer_load_b8(rz, kq * 8 + (col >> 1), (tg[nt] + g_begin + 4 * q) * 8, 0);
      }
  };

  // ---- 2. the activations of this wave's slice of K.  On one stream (no hint word) they are asked for BEFORE the
  // weights: the producer is done, they arrive first and are turned into operands while the weights travel.
  // Otherwise the wave asks (again) until the words carry this step's epoch -- those requests queue behind the wave's
  // weights, which have to arrive anyway. -----------------------------------------------------------------------------
  const int spin_max = a.spin_limit;
  const uint32_t epoch = (uint32_t)*a.epoch, tag16 = epoch & 0xffffu;
  const int k0 = g_begin * 128, k1 = g_end * 128;  // the slice, in elements
  const int nch = (k1 - k0 + 255) >> 8;            // chunks of 256 elements: 4 per lane
  // zero row (operand rows that carry no activation row read it), this wave's slice
  for (int off = k0 * 2 + lane * 16; off < k1 * 2; off += 1024) *reinterpret_cast<u32x4*>(smem + xbytes + off) = u32x4{0u, 0u, 0u, 0u};
  bool gave_up = false;
  if constexpr (MODE == 0) {
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(a.x, (int64_t)K * 2);
    u32x2 v[XC];
#pragma unroll
    for (int c = 0; c < XC; ++c)
      if (c < nch) v[c] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rx, lane * 8, (k0 + c * 256) * 2, 0));
    issue_weights();
#pragma unroll
    for (int c = 0; c < XC; ++c)
      if (c < nch && k0 + c * 256 + lane * 4 < k1) *reinterpret_cast<u32x2*>(smem + (k0 + c * 256 + lane * 4) * 2) = v[c];
  } else {
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(a.x, (int64_t)K * 4);
    const __amdgpu_buffer_rsrc_t rr = make_rsrc(a.resid, MODE == 2 ? (int64_t)K * 4 : 0);
    const __amdgpu_buffer_rsrc_t rn = make_rsrc(a.norm_w, MODE == 2 ? (int64_t)K * 2 : 0);
    const int n_ssq = K >> 4;                       // tagged sums; 256 per request (four per lane)
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(a.ssq_in, MODE == 2 ? (int64_t)n_ssq * 4 : 0);
    constexpr int SL = MODE == 2 ? 2 : 0;           // K <= 8192
    u32x2 nw[XC];
    if constexpr (MODE == 2) {
#pragma unroll
      for (int c = 0; c < XC; ++c)
        if (c < nch) nw[c] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rn, lane * 8, (k0 + c * 256) * 2, 0));
    }
    u32x4 xv[XC], rv[XC], sv[SL > 0 ? SL : 1];
    // Every request goes past the L2 (device-coherent): a line fetched before the producer's stores must never be
    // found there again by a later poll.  (A request that MAY be served by the L2, even one the compiler only
    // speculates, leaves such a line behind, and the device-coherent requests that follow then hit it: the wave
    // sees the old tags until the line happens to be evicted -- measured as waits of a millisecond.)
    auto ask = [&]() {
#pragma unroll
      for (int s = 0; s < SL; ++s)
        if (s * 256 < n_ssq) sv[s] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rq, lane * 16, s * 1024, kSc1));
#pragma unroll
      for (int c = 0; c < XC; ++c)
        if (c < nch) {
          xv[c] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, lane * 16, (k0 + c * 256) * 4, kSc1));
          if constexpr (MODE == 2)
            rv[c] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rr, lane * 16, (k0 + c * 256) * 4, kSc1));
        }
    };
    float ss = 0.f;  // this lane's share of the row's sum of squares (of the last check)
    auto all_tagged = [&]() {  // wave-uniform: every word of the slice carries this step's epoch
      bool ok = true;
      ss = 0.f;
#pragma unroll
      for (int s = 0; s < SL; ++s)
        if (s * 256 + lane * 4 < n_ssq) {  // n_ssq is a multiple of 8 (K of 128)
          ok = ok && sums_ok(sv[s], epoch);
          ss += (sum_of(sv[s].x) + sum_of(sv[s].y)) + (sum_of(sv[s].z) + sum_of(sv[s].w));
        }
#pragma unroll
      for (int c = 0; c < XC; ++c)
        if (c < nch && k0 + c * 256 + lane * 4 < k1) {
          ok = ok && tags_ok(xv[c], tag16);
          if constexpr (MODE == 2) ok = ok && tags_ok(rv[c], tag16);
        }
      return __builtin_amdgcn_ballot_w64(!ok) == 0;
    };
    // With a hint word the launch may be running beside its producer, whose rows are then rarely there yet: a request
    // made now would be wasted traffic (every workgroup asks for the whole row), so the wave asks only once the hint is up.
    const bool eager = a.hint_in == nullptr;
    if (eager) ask();
    issue_weights();
    const bool ready = eager && all_tagged();
    if (a.hint_in && wave == 0 && ready && lane == 0)  // the other waves of the workgroup need not wait for the hint either
      *reinterpret_cast<volatile uint32_t*>(red + WAVES * NT * 16) = epoch ^ (uint32_t)(uintptr_t)a.hint_in;
    if (!ready) {
      int spins = 0, hint_spins = 0;
      // The producer is still at work.  Asking for the whole slice over and over would cost more traffic than the
      // weights (every workgroup reads all of the row), so the wave first watches one word that the producer's last
      // workgroup sets when it is done -- a hint, not a guarantee: the tags decide.
      // One wave per workgroup watches the hint -- one of kHintCopies copies, kHintStride bytes apart, so that the
      // pollers of a launch are spread over the memory channels -- and tells the others through LDS.
      if (a.hint_in) {
        volatile uint32_t* flag = reinterpret_cast<volatile uint32_t*>(red + WAVES * NT * 16);
        const uint32_t mine = epoch ^ (uint32_t)(uintptr_t)a.hint_in;
        if (wave == 0) {
          const __amdgpu_buffer_rsrc_t rh = make_rsrc(a.hint_in, kHintCopies * kHintStride);
          const int copy = (blockIdx.x & (kHintCopies - 1)) * kHintStride;
          for (; spins < spin_max; ++spins) {
            poll_fence();
            if ((uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rh, 0, copy, kSc1) == epoch) break;
            __builtin_amdgcn_s_sleep(16);
          }
          if (lane == 0) *flag = mine;
        } else {
          for (; spins < spin_max; ++spins) {
            poll_fence();
            if (*flag == mine) break;
            __builtin_amdgcn_s_sleep(16);
          }
        }
        hint_spins = spins;
      }
      for (;; ++spins) {
        poll_fence();
        ask();
        if (all_tagged()) break;
        if (spins >= spin_max) {
          gave_up = true;
          break;
        }
        __builtin_amdgcn_s_sleep(4);
      }
      if (a.status[4] && lane == 0) {  // statistics of a tuning run (status[4] set by the host): waits per launch
        atomicMax(a.status + 1, hint_spins);
        atomicMax(a.status + 2, spins - hint_spins);
        atomicAdd(a.status + 3, 1);
      }
    }
    float rstd = 0.f;
    if constexpr (MODE == 2)  // 1 / rms of the row: the per-tile partials in a fixed order (lane-strided, then the tree)
      rstd = 1.f / sqrtf(wave_sum(ss) / (float)K + a.eps);
    const __amdgpu_buffer_rsrc_t ro = make_rsrc(a.x_out, MODE == 2 ? (int64_t)K * 4 : 0);
#pragma unroll
    for (int c = 0; c < XC; ++c)
      if (c < nch) {
        const int e = k0 + c * 256 + lane * 4;
        u32x2 o = untag4(xv[c]);
        if constexpr (MODE == 2) {  // resid + w * round(a * rstd), rounding points of olmo/model.py:241-255 and the bf16 add
          const u32x2 r = untag4(rv[c]);
          float f[4] = {bf16lo_to_f32(o.x), bf16hi_to_f32(o.x), bf16lo_to_f32(o.y), bf16hi_to_f32(o.y)};
          const float rr4[4] = {bf16lo_to_f32(r.x), bf16hi_to_f32(r.x), bf16lo_to_f32(r.y), bf16hi_to_f32(r.y)};
          const float ww[4] = {bf16lo_to_f32(nw[c].x), bf16hi_to_f32(nw[c].x), bf16lo_to_f32(nw[c].y), bf16hi_to_f32(nw[c].y)};
#pragma unroll
          for (int i = 0; i < 4; ++i) f[i] = round_bf16(rr4[i] + round_bf16(ww[i] * round_bf16(f[i] * rstd)));
          o = u32x2{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3])};
          if (blockIdx.x == 0 && e < k1) {
            const u32x4 t = {tag_word(f[0], tag16), tag_word(f[1], tag16), tag_word(f[2], tag16), tag_word(f[3], tag16)};
            __builtin_amdgcn_raw_buffer_store_b128(t, ro, lane * 16, (k0 + c * 256) * 4, kSc1);
          }
        }
        if (e < k1) *reinterpret_cast<u32x2*>(smem + e * 2) = o;
      }
  }
  if (gave_up && lane == 0) {
    __hip_atomic_store(a.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (a.status[4]) atomicOr(a.status + 5, 1 << MODE), atomicAdd(a.status + 6, 1);
  }

  // ---- 3. the products: one accumulator per quad of groups, group u of the quad in operand rows 4u (row 0 = the
  // activation row, the others the zero row), so its products land in the lanes of row block u ---------------------
  int xoff[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) xoff[u] = (col == 4 * u ? 0 : K) + 8 * kq;
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const bf16x8 ones = ones_bf16x8();
  const UnpackConsts uc;
  float acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt] = 0.f;
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    f32x4 t[NT], xsum = zero4;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) t[nt] = zero4;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int g = g_begin + 4 * q + u;
      if (g < g_end) {
        const uint16_t* xp = xl + xoff[u] + 128 * g;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bf16x8 af = *reinterpret_cast<const bf16x8*>(xp + 32 * j);
          xsum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, ones, xsum, 0, 0, 0);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            t[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, unpack_w4_bias128(w[q][u][nt][j], uc), t[nt], 0, 0, 0);
        }
      }
    }
    // fp32 correction acc += scale * (T - (128 + zero) * X); a row block whose group lies past the wave's share holds zeros
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const float sc = (float)__builtin_bit_cast(_Float16, (uint16_t)s16[q][nt]);
      const float nzc = -(float)(129 + (int)((z8[q][nt] >> (4 * (col & 1))) & 15u));  // -(128 + (stored + 1))
      acc[nt] = __builtin_fmaf(sc, __builtin_fmaf(nzc, xsum[0], t[nt][0]), acc[nt]);
    }
  }

  // ---- 4. the four row blocks inside the wave, then the waves through LDS, in a fixed order ------------------------
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    float v = acc[nt];
    v = combine_xor16(v, AddOp{});
    v = combine_xor32(v, AddOp{});
    if (kq == 0) red[(wave * NT + nt) * 16 + col] = v;
  }
  // the tagged residual row of workgroup 0 has landed before anything of this launch's output can be seen
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));
  __syncthreads();
  auto total_of = [&](int nt, int c) {
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) v += red[(wv * NT + nt) * 16 + c];
    return v;
  };
  if (a.hint_out && blockIdx.x == gridDim.x - 1 && tid < kHintCopies)
    __hip_atomic_store(a.hint_out + tid * (kHintStride / 4), (int32_t)epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if constexpr (EPI == 0) {
    if (tid < NT * 16) {
      const int c = tid & 15, nt = tid >> 4;
      const bool live = tile[nt] < ntiles;
      const float v = live ? round_bf16(total_of(nt, c)) : 0.f;
      const int n = tile[nt] * 16 + c;
      if (live) {
        if (a.y_tagged) __hip_atomic_store(reinterpret_cast<uint32_t*>(a.y) + n, tag_word(v, tag16), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else reinterpret_cast<uint16_t*>(a.y)[n] = f32_to_bf16_bits(v);
      }
      if (a.ssq_out) {  // sum of squares of the tile's 16 outputs: one row of 16 lanes
        const float qv = row16_sum(v * v);
        if (live && c == 0)
          __hip_atomic_store(a.ssq_out + tile[nt], tag_sum(qv, epoch), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  } else {
    if (tid < 16) {
      const float up = round_bf16(total_of(0, tid));  // the Linear's bf16 output
      const float gate = round_bf16(total_of(1, tid));
      const float sg = round_bf16(gate / (1.f + expf(-gate)));
      const float v = round_bf16(sg * up);
      const int n = tile[0] * 16 + tid;
      if (a.y_tagged) __hip_atomic_store(reinterpret_cast<uint32_t*>(a.y) + n, tag_word(v, tag16), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else reinterpret_cast<uint16_t*>(a.y)[n] = f32_to_bf16_bits(v);
    }
  }
}

// out = resid + rmsnorm(x; norm_w) for one tagged row (the last block's pending update, olmo/model.py:814-821),
// written as plain bf16 for the launches after the relay.  One workgroup.
__global__ __launch_bounds__(256) void relay_final_kernel(const uint32_t* __restrict__ x, const uint32_t* __restrict__ ssq_in,
                                                          const uint32_t* __restrict__ resid, const uint16_t* __restrict__ norm_w,
                                                          uint16_t* __restrict__ out, int K, float eps,
                                                          const int32_t* __restrict__ epoch_p, int32_t* status, int spin_limit) {
  __shared__ float part[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t epoch = (uint32_t)*epoch_p, tag16 = epoch & 0xffffu;
  const int n_ssq = K >> 4;
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(x, (int64_t)K * 4), rr = make_rsrc(resid, (int64_t)K * 4),
                               rq = make_rsrc(ssq_in, (int64_t)n_ssq * 4);
  constexpr int C = 8;  // K <= 8192: 1024 elements per pass of the workgroup
  u32x4 xv[C], rv[C], sv;
  bool gave_up = false;
  for (int spins = 0;; ++spins) {
    bool ok = true;
    poll_fence();
    sv = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rq, tid * 16, 0, kSc1));  // 512 sums at most: four per thread
    if (tid * 4 < n_ssq) ok = ok && sums_ok(sv, epoch);
#pragma unroll
    for (int c = 0; c < C; ++c)
      if (c * 1024 < K) {
        xv[c] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, tid * 16, c * 4096, kSc1));
        rv[c] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rr, tid * 16, c * 4096, kSc1));
        if (c * 1024 + tid * 4 < K) ok = ok && tags_ok(xv[c], tag16) && tags_ok(rv[c], tag16);
      }
    if (__syncthreads_and(ok)) break;
    if (spins >= spin_limit) {
      gave_up = true;
      break;
    }
    __builtin_amdgcn_s_sleep(4);
  }
  if (gave_up && tid == 0) {
    __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (status[4]) atomicOr(status + 5, 16);
  }
  float ss = 0.f;
  if (tid * 4 < n_ssq) ss = (sum_of(sv.x) + sum_of(sv.y)) + (sum_of(sv.z) + sum_of(sv.w));
  ss = wave_sum(ss);
  if (lane == 0) part[wave] = ss;
  __syncthreads();
  const float rstd = 1.f / sqrtf(((part[0] + part[1]) + (part[2] + part[3])) / (float)K + eps);
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int e = c * 1024 + tid * 4;
    if (e < K) {
      const u32x2 xa = untag4(xv[c]), r = untag4(rv[c]);
      const u32x2 nw = *reinterpret_cast<const u32x2*>(norm_w + e);
      const float f[4] = {bf16lo_to_f32(xa.x), bf16hi_to_f32(xa.x), bf16lo_to_f32(xa.y), bf16hi_to_f32(xa.y)};
      const float rr4[4] = {bf16lo_to_f32(r.x), bf16hi_to_f32(r.x), bf16lo_to_f32(r.y), bf16hi_to_f32(r.y)};
      const float ww[4] = {bf16lo_to_f32(nw.x), bf16hi_to_f32(nw.x), bf16lo_to_f32(nw.y), bf16hi_to_f32(nw.y)};
      float o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = rr4[i] + round_bf16(ww[i] * round_bf16(f[i] * rstd));
      *reinterpret_cast<u32x2*>(out + e) = u32x2{pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
    }
  }
}

// plain bf16 row -> tagged words (the relay's first residual row: the embedding of the step's token)
__global__ __launch_bounds__(256) void relay_tag_kernel(const uint16_t* __restrict__ x, uint32_t* __restrict__ out, int n,
                                                        const int32_t* __restrict__ epoch_p) {
  const uint32_t tag16 = (uint32_t)*epoch_p & 0xffffu;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) __hip_atomic_store(out + i, ((uint32_t)x[i] << 16) | tag16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- launch plans ------------------------------------------------------------------------------------------------
struct RelayCfg {
  int waves, nt, nq;
};

// the smallest number of quads that holds a wave's share of K
inline int quads_for(int K, int waves) { return ((((K >> 7) + waves - 1) / waves) + 3) / 4; }

// cfg: 0 = choose, else waves | nt << 8 (nq follows from K and waves)
inline bool relay_cfg(int N, int K, int swiglu, int cfg, RelayCfg* out) {
  const int ntiles = N >> 4;
  RelayCfg c;
  if (cfg) {
    c.waves = cfg & 0xff, c.nt = (cfg >> 8) & 0xff;
  } else {
    // narrow outputs: one tile per workgroup, K over 16 waves; wide ones: 8 waves (measured on the 7B shapes)
    c.waves = ntiles <= 512 ? 16 : 8;
    c.nt = 1;
  }
  if (swiglu) c.nt = 2;
  if (c.waves != 4 && c.waves != 8 && c.waves != 16) return false;
  if (c.nt != 1 && c.nt != 2) return false;
  c.nq = quads_for(K, c.waves);
  while (!cfg && c.nq > 3 && c.waves < 16) c.waves *= 2, c.nq = quads_for(K, c.waves);
  if (c.nq < 1 || c.nq > 3) return false;
  *out = c;
  return true;
}

inline size_t relay_lds(int K, const RelayCfg& c) { return (size_t)4 * K + (size_t)c.waves * c.nt * 16 * 4 + 16; }  // + the hint flag

template <typename F>
int with_relay_kernel(const RelayCfg& c, int mode, int swiglu, F&& f) {
#define RELAY_CASE(NTv, Wv, NQv, MODEv, EPIv)                                                          \
  if (c.nt == NTv && c.waves == Wv && c.nq == NQv && mode == MODEv && swiglu == EPIv)                  \
    return f(w4_relay_kernel<NTv, Wv, NQv, MODEv, EPIv>);
#define RELAY_SHAPES(MODEv, NTv, EPIv)                                                                                        \
  RELAY_CASE(NTv, 4, 1, MODEv, EPIv) RELAY_CASE(NTv, 4, 2, MODEv, EPIv) RELAY_CASE(NTv, 4, 3, MODEv, EPIv)                    \
  RELAY_CASE(NTv, 8, 1, MODEv, EPIv) RELAY_CASE(NTv, 8, 2, MODEv, EPIv) RELAY_CASE(NTv, 8, 3, MODEv, EPIv)                    \
  RELAY_CASE(NTv, 16, 1, MODEv, EPIv) RELAY_CASE(NTv, 16, 2, MODEv, EPIv)
  RELAY_SHAPES(0, 1, 0) RELAY_SHAPES(0, 2, 0)
  RELAY_SHAPES(1, 1, 0) RELAY_SHAPES(1, 2, 0)
  RELAY_SHAPES(2, 1, 0) RELAY_SHAPES(2, 2, 0)
  RELAY_SHAPES(2, 2, 1)
#undef RELAY_SHAPES
#undef RELAY_CASE
  return O355_EUNSUPPORTED;
}

int relay_check(const void* x, int x_tagged, const uint32_t* ssq_in, const uint32_t* resid, const uint16_t* norm_w,
                const uint32_t* x_out, const void* wt, const void* st, const void* zt, const void* y, int N, int K,
                int swiglu, const int32_t* epoch, const int32_t* status, int spin_limit, int* mode) {
  if (!x || !wt || !st || !zt || !y || !epoch || !status || N <= 0 || K <= 0 || spin_limit < 0) return O355_EINVAL;
  const bool norm = resid != nullptr;
  if (norm && (!ssq_in || !norm_w || !x_out || !x_tagged)) return O355_EINVAL;
  if (!norm && (ssq_in || norm_w || x_out)) return O355_EINVAL;
  if ((K & 127) || (N & (swiglu ? 31 : 15)) || K > 8192 * (norm ? 1 : 3)) return O355_EUNSUPPORTED;
  if ((int64_t)(N >> 4) * (K >> 7) * 1024 >= (1ll << 31)) return O355_EUNSUPPORTED;
  if (swiglu && !norm) return O355_EUNSUPPORTED;
  *mode = norm ? 2 : (x_tagged ? 1 : 0);
  return O355_OK;
}

}  // namespace

extern "C" int olmo355_w4_relay(const void* x, int x_tagged, const uint32_t* ssq_in, const uint32_t* resid,
                                const uint16_t* norm_w, float eps, uint32_t* x_out, const uint32_t* wt, const uint16_t* st,
                                const uint8_t* zt, void* y, int y_tagged, uint32_t* ssq_out, int N, int K, int swiglu,
                                const int32_t* epoch, int32_t* status, const int32_t* hint_in, int32_t* hint_out,
                                int spin_limit, int cfg, void* stream) {
  int mode = 0;
  const int chk = relay_check(x, x_tagged, ssq_in, resid, norm_w, x_out, wt, st, zt, y, N, K, swiglu, epoch, status, spin_limit, &mode);
  if (chk != O355_OK) return chk;
  if (swiglu && ssq_out) return O355_EUNSUPPORTED;
  RelayCfg c;
  if (!relay_cfg(N, K, swiglu, cfg, &c)) return O355_EUNSUPPORTED;
  RelayArgs a{x, ssq_in, resid, norm_w, x_out, y, ssq_out, epoch, status, hint_in, hint_out, eps, N, K, x_tagged, y_tagged, spin_limit};
  const size_t lds = relay_lds(K, c);
  const int ntiles = N >> 4;
  const unsigned blocks = swiglu ? (unsigned)(ntiles >> 1) : (unsigned)((ntiles + c.nt - 1) / c.nt);
  return with_relay_kernel(c, mode, swiglu ? 1 : 0, [&](auto kern) {
    if (lds > 48 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return (int)O355_ELAUNCH;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(c.waves * 64), lds, as_stream(stream), a, (const u32x4*)wt, st, zt);
    return hipGetLastError() == hipSuccess ? (int)O355_OK : (int)O355_ELAUNCH;
  });
}

// What a launch of olmo355_w4_relay takes of the chip: out[0] workgroups, out[1] waves per workgroup, out[2] vector
// registers per lane, out[3] bytes of LDS per workgroup.
extern "C" int olmo355_w4_relay_footprint(int N, int K, int norm, int x_tagged, int swiglu, int cfg, int* out) {
  if (!out || N <= 0 || K <= 0) return O355_EINVAL;
  RelayCfg c;
  if (!relay_cfg(N, K, swiglu, cfg, &c)) return O355_EUNSUPPORTED;
  const int mode = norm ? 2 : (x_tagged ? 1 : 0);
  const int ntiles = N >> 4;
  out[0] = swiglu ? (ntiles >> 1) : (ntiles + c.nt - 1) / c.nt;
  out[1] = c.waves;
  out[3] = (int)relay_lds(K, c);
  return with_relay_kernel(c, mode, swiglu ? 1 : 0, [&](auto kern) {
    hipFuncAttributes fa;
    if (hipFuncGetAttributes(&fa, reinterpret_cast<const void*>(kern)) != hipSuccess) return (int)O355_ELAUNCH;
    out[2] = fa.numRegs;
    out[3] += (int)fa.sharedSizeBytes;
    return (int)O355_OK;
  });
}

// Whether a launch B (the younger one, which may wait for A's output) can never keep a workgroup of A from
// starting: with n workgroups of B on a CU one of A must still fit, for every n that B's grid can put on all CUs
// at once.  Footprints as olmo355_w4_relay_footprint returns them.  CU: 4 SIMDs of 8 wave slots and 512 vector
// registers per lane (allocated in blocks of 8), `lds_per_cu` bytes of LDS (allocated in blocks of 1 KiB here,
// which over-estimates).
extern "C" int olmo355_relay_pair_ok(const int* a, const int* b, int n_cu, int lds_per_cu) {
  if (!a || !b || n_cu <= 0 || lds_per_cu <= 0) return 0;
  auto per_simd = [](int waves) { return (waves + 3) / 4; };
  auto regs = [](int r) { return (std::max(r, 1) + 7) / 8 * 8; };
  auto lds = [](int l) { return (l + 1023) / 1024 * 1024; };
  const int wa = per_simd(a[1]), wb = per_simd(b[1]);
  int n = 0;  // workgroups of B on a CU next to which one of A still fits
  for (;; ++n) {
    const bool fits = n * wb + wa <= 8 && n * wb * regs(b[2]) + wa * regs(a[2]) <= 512 && n * lds(b[3]) + lds(a[3]) <= lds_per_cu;
    if (!fits) break;
    if (n > 64) return 1;  // B is tiny
  }
  // n is the smallest count that blocks A on a CU; B can do that on every CU only with n * n_cu workgroups
  return n > 0 && (int64_t)b[0] < (int64_t)n * n_cu ? 1 : 0;
}

// out[0] = CUs of the current device, out[1] = bytes of LDS per CU: the chip side of olmo355_relay_pair_ok
extern "C" int olmo355_relay_device(int* out) {
  int dev = 0, cus = 0, lds = 0;
  if (!out) return O355_EINVAL;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev) != hipSuccess || cus <= 0 || lds <= 0)
    return O355_ELAUNCH;
  out[0] = cus, out[1] = lds;
  return O355_OK;
}

extern "C" int olmo355_relay_final(const uint32_t* x, const uint32_t* ssq_in, const uint32_t* resid, const uint16_t* norm_w,
                                   float eps, uint16_t* out, int K, const int32_t* epoch, int32_t* status, int spin_limit,
                                   void* stream) {
  if (!x || !ssq_in || !resid || !norm_w || !out || !epoch || !status || K <= 0 || spin_limit < 0) return O355_EINVAL;
  if ((K & 15) || K > 8192) return O355_EUNSUPPORTED;
  hipLaunchKernelGGL(relay_final_kernel, dim3(1), dim3(256), 0, as_stream(stream), x, ssq_in, resid, norm_w, out, K, eps, epoch,
                     status, spin_limit);
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_relay_tag(const uint16_t* x, uint32_t* out, int n, const int32_t* epoch, void* stream) {
  if (!x || !out || !epoch || n <= 0) return O355_EINVAL;
  hipLaunchKernelGGL(relay_tag_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream), x, out, n, epoch);
  O355_CHECK_LAUNCH();
}
