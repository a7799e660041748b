// Causal attention over the contiguous per-layer KV cache [B, Hkv, Lmax, hd]
// (olmo/model.py:533-586,627-648): softmax(q k^T / sqrt(hd) + bias) v, fp32 softmax.
//
//  * attn_prefill_mfma_kernel  bf16, hd 64/128: flash-style, K tiles in LDS in MFMA-fragment order and V
//    tiles row-major (read with transposing loads), both loaded memory -> LDS directly a tile ahead;
//    S^T = K.Q^T and O^T = V^T.P^T on the matrix cores so the softmax statistics of a query stay in
//    one lane column and P never leaves registers.
//  * attn_decode_kernel        one query per sequence, keys split over workgroups and waves,
//    DPP / wave reductions, partial (max, sum, o) merged by attn_decode_combine_kernel.
//  * attn_generic_kernel       any dtype / head size <= 128, one query per thread (used for the
//    fp32 model configuration).
//
// Masking: keys after the query position are skipped.  A key whose key_bias entry is <= -1e30
// (padding) keeps a *finite* score, the dtype's most negative value, as in the reference
// (olmo/model.py:1337-1376, olmo/torch_util.py:81-90): a query that sees only padding gets a
// plain average of values instead of NaN -- in the reference over every key of the call, which
// attn_masked_rows_kernel reproduces after a prefill launch; a decode step's single query (a real
// token, never masked itself) needs no such pass.
#include "common.h"
#include "../../include/olmo355_debug.h"

#include <mutex>
#include <type_traits>

namespace {

constexpr float kMaskThreshold = -1e30f;
constexpr float kLazyMax = 8.f;

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
template <> struct Vec8<O355_F16> {
  static __device__ __forceinline__ void unpack(const u32x4 (&r)[1], float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f16x2 h = __builtin_bit_cast(f16x2, (uint32_t)r[0][i]);
      f[2 * i] = (float)h[0], f[2 * i + 1] = (float)h[1];
    }
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
// Workgroup: 4 waves x 32 queries = 128 queries of one (batch, head); KV tile: 64 keys, two tiles in LDS: the
// tile after the one being multiplied travels memory -> LDS directly while that goes on, one barrier per tile.
// The LDS side of such a load is lane-linear (64 lanes x 16 bytes = 1 KiB per instruction), so the layouts below
// are produced on the memory side, by which 16 bytes each lane asks for.
// LDS  K  : [key-tile 4][hd-step HD/32][64 lanes][8 bf16]   A operand of S^T = K . Q^T, one conflict-free
//           ds_read_b128 per fragment
//      V  : [key 64][hd] row-major, rows HD * 2 bytes apart, the 32-byte units of a row XOR-swizzled by the key so
//           that 8 neighbouring keys' units of one channel block cover all 64 banks.  The A operand of
//           O^T = V^T . P^T is read with the LDS transposing load (ds_read_b64_tr_b16): per group of 16 lanes,
//           lane r supplies the address of four consecutive bf16 and lane j receives element j % 4 of the four
//           rows supplied by lanes j / 4 + 4 e (e = 0 .. 3).  With lane r pointing at key 4 kq + r / 4, channels
//           4 (r % 4) .. + 3 of the hd tile, lane j receives channel j of keys 4 kq .. 4 kq + 3: one load per
//           half of an operand fragment, no shuffling of V on the way into LDS.
// In the second product the 8 key slots of lane group kq in key-step s are
//   e<4 : key 32s + 4kq + e        e>=4 : key 32s + 16 + 4kq + (e-4)
// which is exactly how the S^T accumulators of the two 16-key tiles 2s, 2s+1 sit in a lane, so
// P goes from accumulator registers to the B operand without leaving the lane.
// The prefill kernel's reductions over the four lane groups that share a query column: op over l ^ 16, then over
// l ^ 32 (register swaps, see combine_xor16 / combine_xor32).
template <typename Op>
__device__ __forceinline__ float reduce_lane_groups(float v, Op op) {
  return combine_xor32(combine_xor16(v, op), op);
}

// One wave's requests for a K / V tile of the prefill kernel: HD / 32 instructions of 1 KiB per operand, memory ->
// LDS directly (kdst / vdst: the wave's first KiB of the tile's buffers).  row: key within the tile, in: byte
// within the key's row, per instruction and lane.  Only the last tile can reach past the last visible key; rows
// past it may hold anything, so the last visible row is read in their place.
// (A function and not a lambda of the kernel: with the memory -> LDS builtin inside a lambda that the kernel calls,
// this toolchain's host pass emits no launch stub for the kernel, without a diagnostic, and the library then fails
// to load with an undefined symbol.)
template <int S>  // S = HD / 32, deduced from the arrays
__device__ __forceinline__ void prefill_request_tile(__amdgpu_buffer_rsrc_t rk, __amdgpu_buffer_rsrc_t rv, unsigned char* kdst,
                                                     unsigned char* vdst, const int (&k_row)[S], const int (&k_in)[S],
                                                     const int (&v_row)[S], const int (&v_in)[S], int k0, int last_pos) {
  constexpr int HD = 32 * S;
  const bool tail = k0 + 63 > last_pos;
#pragma unroll
  for (int i = 0; i < HD / 32; ++i) {
    const int kr = tail ? min(k0 + k_row[i], last_pos) - k0 : k_row[i];
    const int vr = tail ? min(k0 + v_row[i], last_pos) - k0 : v_row[i];
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (lds_ptr_t)(kdst + (i << 10)), 16, kr * (HD * 2) + k_in[i], k0 * (HD * 2), 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (lds_ptr_t)(vdst + (i << 10)), 16, vr * (HD * 2) + v_in[i], k0 * (HD * 2), 0, 0);
  }
}

template <int HD>
struct PrefillLds {
  static constexpr int KT = 64;
  static constexpr int TILE = KT * HD * 2;            // bytes of one K (or V) tile
  static constexpr int BYTES = 4 * TILE + 2 * KT * 4;  // K x 2, V x 2, bias x 2
};

// SPLIT (past_len == 0, at most kPrefillMaxChunks x chunk_blocks query blocks): a query block whose keys run
// past chunk_blocks x 128 is shared by several workgroups, one per run of that many keys.  One prompt of 2048
// tokens and 16 heads is 256 workgroups of 1 to 16 units of work each for the chip's 512 places: the launch lasts as
// long as its longest workgroup while most places stand empty; cut at 8 units the same work is 384 workgroups of at
// most half that length, all resident at once.  A workgroup that does not hold all of its block's keys
// leaves its accumulators, reference maximum and denominator as they stand in its slot of the workspace
// (device-scope stores) and draws a ticket; the one that draws the block's last ticket adds the others' to its own
// registers and writes the output.  Nobody waits for anybody.
constexpr int kPrefillMaxChunks = 4;
constexpr int kPrefillMaxTriples = 1024, kPrefillTicketBytes = 4096;  // (batch, head, query block) triples of a split launch
template <int HD>
struct PrefillSplit {
  static constexpr int O_BYTES = 4 * 2 * (HD / 16) * 64 * 16;  // waves x query tiles x channel tiles x lanes x float4
  static constexpr int ML_BYTES = 4 * 2 * 64 * 8;              // (reference maximum, denominator) per wave, query tile, lane
  static constexpr int SLOT_BYTES = O_BYTES + ML_BYTES;
};

template <int HD>
__global__ __launch_bounds__(256, 2) void attn_prefill_mfma_kernel(const uint16_t* __restrict__ q,
                                                                const uint16_t* __restrict__ kc,
                                                                const uint16_t* __restrict__ vc,
                                                                const float* __restrict__ key_bias,
                                                                uint16_t* __restrict__ out, int T, int H, int Hkv,
                                                                int Lmax, int past_len, int bias_stride,
                                                                unsigned char* __restrict__ ws, int max_chunks, int chunk_blocks) {
  const bool SPLIT = ws != nullptr;  // uniform over the launch
  const int kPrefillChunkBlocks = chunk_blocks;  // query blocks' worth of keys (x 128) per run
  constexpr int KT = 64;             // keys per tile
  constexpr int STEPS = HD / 32;     // hd steps of the first product = 1 KiB load instructions per wave, tile and operand
  constexpr int HT = HD / 16;        // hd tiles of the second product
  constexpr int QT = 2;              // 16-query tiles per wave
  constexpr int TILE = PrefillLds<HD>::TILE;
  constexpr int CPR = HD / 8;        // 16-byte chunks per key row
  constexpr int VROW = HD * 2;       // bytes per key row of V in LDS
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* const lds_k = smem;             // [2][TILE]
  unsigned char* const lds_v = smem + 2 * TILE;  // [2][TILE]
  float* const lds_bias = reinterpret_cast<float*>(smem + 4 * TILE);  // [2][KT]

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  // One 128-query block per workgroup, two workgroups per CU.  Causal work grows with the block index;
  // blockIdx.y is the rank in this order: the heaviest half of the blocks (descending), then the
  // lightest half (ascending), so the two workgroups a CU holds -- rank r and rank r + nqb/2 when the
  // grid just fills the chip, heads varying fastest -- add up to about the same number of key tiles.
  const int nqb = (T + 127) / 128;
  const int b = blockIdx.z, h = blockIdx.x, hk = h / (H / Hkv);
  const float lowest = -3.3895313892515355e38f;
  const float c2 = 1.4426950408889634f / sqrtf((float)HD);  // scores live in the log2 domain: exp2(s*c2 + bias*log2e - m)
  const int64_t cbase = ((int64_t)b * Hkv + hk) * Lmax * HD;
  const int half = (nqb + 1) / 2, rank = blockIdx.y;
  int qblock = rank < half ? nqb - 1 - rank : rank - half;
  int chunk = 0, nchunks = 1;
  if (SPLIT) {
    // blockIdx.y counts the (block, run of keys) pairs longest first: the full runs (block b has b / CB of them), then
    // the blocks' last runs by length, CB units down to 1 (block b's last run is b % CB + 1 units long)
    const int CB = kPrefillChunkBlocks;
    int r = rank;
    qblock = -1;
    for (int bb = nqb - 1; bb >= CB && qblock < 0; --bb) {
      const int f = bb / CB;
      if (r < f) qblock = bb, chunk = r;
      else r -= f;
    }
    for (int sz = CB; sz >= 1 && qblock < 0; --sz) {
      const int cnt = sz - 1 < nqb ? (nqb - (sz - 1) + CB - 1) / CB : 0;
      if (r < cnt) qblock = sz - 1 + r * CB, chunk = qblock / CB;
      else r -= cnt;
    }
    nchunks = qblock / CB + 1;
  }
  const int q0 = qblock * 128 + wave * 32;

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
  float m[QT], l[QT];  // l: this lane's share of the denominator (its 16 of a tile's 64 keys); added up at the end
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    m[qt] = -INFINITY, l[qt] = 0.f;
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) o[qt][ht] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int last_pos = past_len + min(qblock * 128 + 127, T - 1);   // workgroup-uniform loop bound
  const int wave_last = past_len + min(q0 + 31, T - 1);             // last position this wave needs
  // range-checked loads: the tile's base as the scalar offset, a lane's place in the tile worked out once.
  // Wave w asks for the K fragments of key tile w (one instruction per hd step) and for V rows
  // w * KT / 4 .. + KT / 4 - 1 (STEPS instructions of 1 KiB).
  const __amdgpu_buffer_rsrc_t rk_ = make_rsrc(kc + cbase, (int64_t)Lmax * HD * 2);
  const __amdgpu_buffer_rsrc_t rv_ = make_rsrc(vc + cbase, (int64_t)Lmax * HD * 2);
  auto v_swz = [](int key) { return HD == 128 ? (key & 7) : ((key >> 1) & 3); };  // on the 32-byte units of a row
  int k_row[STEPS], k_in[STEPS], v_row[STEPS], v_in[STEPS];  // key within the tile, byte within the row
#pragma unroll
  for (int i = 0; i < STEPS; ++i) {
    k_row[i] = 16 * wave + col;
    k_in[i] = (4 * i + kq) * 16;
    const int slot = (wave * STEPS + i) * 64 + lane;  // 16-byte slot of the V tile this lane fills
    const int row = slot / CPR, pos = slot % CPR;
    v_row[i] = row;
    v_in[i] = ((((pos >> 1) ^ v_swz(row)) << 1) | (pos & 1)) * 16;
  }
  float rbias = 0.f;
  auto fetch = [&](int k0, int buf) {
    prefill_request_tile(rk_, rv_, lds_k + buf * TILE + wave * (STEPS << 10), lds_v + buf * TILE + wave * (STEPS << 10), k_row,
                             k_in, v_row, v_in, k0, last_pos);
    if (key_bias && tid < KT) rbias = key_bias[(int64_t)b * bias_stride + min(k0 + tid, last_pos)];
  };
  auto publish = [&](int buf) {  // own requests landed, then everybody's
    if (tid < KT) lds_bias[buf * KT + tid] = rbias;  // zeros without a key_bias: the diagonal tiles read it either way
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, true));
    __builtin_amdgcn_s_barrier();
  };
  // this lane's row of the transposing loads, per hd tile (the swizzle of the lane's keys is the same for every
  // key step: they differ by multiples of 16)
  int v_rd[HT];
#pragma unroll
  for (int ht = 0; ht < HT; ++ht) v_rd[ht] = (4 * kq + (col >> 2)) * VROW + ((ht ^ v_swz(4 * kq + (col >> 2))) << 5) + 8 * (col & 3);
  const int k_first = SPLIT ? chunk * (kPrefillChunkBlocks * 128) : 0;
  const int k_last = SPLIT ? min(last_pos, k_first + kPrefillChunkBlocks * 128 - 1) : last_pos;  // this workgroup's run of keys
  fetch(k_first, 0);
  publish(0);
  int buf = 0;
  for (int k0 = k_first; k0 <= k_last; k0 += KT, buf ^= 1) {
    // the other buffer was read during the previous tile, and everybody is past that tile's barrier
    if (k0 + KT <= k_last) fetch(k0 + KT, buf ^ 1);
    if (k0 <= wave_last) {  // else nothing visible to this wave in the tile (barriers stay uniform)
    const u32x4* kt_ = reinterpret_cast<const u32x4*>(lds_k + buf * TILE);
    const unsigned char* vt_ = lds_v + buf * TILE;
    const float* bias_ = lds_bias + buf * KT;

    // ---- S^T = K . Q^T -----------------------------------------------------------------------------
    // all of the tile's K fragments are asked for before the first product, so that only the first waits out the
    // LDS latency
    f32x4 s[QT][4];
    u32x4 kf[4 * STEPS];
#pragma unroll
    for (int i = 0; i < 4 * STEPS; ++i) kf[i] = kt_[i * 64 + lane];
    __builtin_amdgcn_sched_barrier(0);  // or the scheduler moves each read down to its use
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
      for (int st = 0; st < STEPS; ++st) {
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
          s[qt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf[kt * STEPS + st]), qf[qt][st],
                                                              st == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : s[qt][kt], 0, 0, 0);
      }
    }
    // ---- online softmax per query column, in the log2 domain -----------------------------------------------
    // Only tiles that reach past the wave's first query need the causal compare, and only calls with a
    // padding bias need the bias terms: the common tile costs a max, one fma and one exp2 per score.
    const bool masked = key_bias != nullptr || k0 + KT - 1 > past_len + q0;  // wave-uniform
    const float cs = masked ? 1.f : c2;  // the masked path leaves its scores already scaled
    bf16x8 pf[QT][2];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      float tmax = -INFINITY;
      if (masked) {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int kk = kt * 16 + 4 * kq + r;
            const float bias = bias_[kk];
            float v = bias <= kMaskThreshold ? lowest : __builtin_fmaf(s[qt][kt][r], c2, bias * 1.4426950408889634f);
            v = k0 + kk > qpos[qt] ? -INFINITY : v;
            s[qt][kt][r] = v;
            tmax = fmaxf(tmax, v);
          }
      } else {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int r = 0; r < 4; ++r) tmax = fmaxf(tmax, s[qt][kt][r]);
        tmax *= c2;  // c2 > 0: the maximum commutes with the scaling
      }
      // The reference maximum follows the running maximum lazily: it moves only when the tile's maximum is more than
      // kLazyMax (log2 units) above it, so probabilities stay below 2^kLazyMax and the accumulators are rescaled
      // on a few tiles instead of nearly all (the same ratio o / l comes out; finite: key 0 of the first tile is
      // visible to every query, and -inf + kLazyMax is -inf).  m is the same in the four lane groups of a query
      // column, so when no lane's own maximum is that far above it the column's is not either, and the exchange
      // between the lane groups is skipped with the rescaling.
      if (__builtin_amdgcn_ballot_w64(tmax > m[qt] + kLazyMax) != 0) {
        tmax = reduce_lane_groups(tmax, [](float a, float b) { return fmaxf(a, b); });
        const float mn = tmax > m[qt] + kLazyMax ? tmax : m[qt];
        const float alpha = __builtin_amdgcn_exp2f(m[qt] - mn);  // 1 where the column's maximum stays
        l[qt] *= alpha;
#pragma unroll
        for (int ht = 0; ht < HT; ++ht)
#pragma unroll
          for (int r = 0; r < 4; ++r) o[qt][ht][r] *= alpha;
        m[qt] = mn;
      }
      const float mn = m[qt];
      float psum = 0.f;
      float p[4][4];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          p[kt][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[qt][kt][r], cs, -mn));
          psum += p[kt][r];
        }
      l[qt] += psum;
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
    // all of the tile's V fragments are asked for before the first product (the compiler lets the first of these
    // loads wait for the outstanding memory -> LDS requests: it cannot tell that they fill the other buffer; written
    // as assembly with hand-placed waits the loads lose that wait and the kernel runs no faster)
    bf16x8 vf[HT][2];
#pragma unroll
    for (int ht = 0; ht < HT; ++ht)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        typedef short s16x4 __attribute__((ext_vector_type(4)));
        typedef s16x4 __attribute__((address_space(3))) * tr_ptr;
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        const unsigned char* vp = vt_ + v_rd[ht] + (32 * s2) * VROW;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)vp);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(vp + 16 * VROW));
        vf[ht][s2] = __builtin_bit_cast(bf16x8, s16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
      }
    __builtin_amdgcn_sched_barrier(0);  // or the scheduler moves each load down to its use
#pragma unroll
    for (int ht = 0; ht < HT; ++ht)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) o[qt][ht] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[ht][s2], pf[qt][s2], o[qt][ht], 0, 0, 0);
    }
    publish(buf ^ 1);  // the next tile is in LDS and this one has been read by everybody
  }
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) l[qt] = reduce_lane_groups(l[qt], [](float a, float b) { return a + b; });
  if (SPLIT) {
    if (nchunks > 1) {
      using PS = PrefillSplit<HD>;
      // the workspace: one ticket counter per (batch, head, block), then the slots [batch][head][block - 8][run]
      // (the counters' region has one size for every shape: a workspace that served another shape must not be
      // found holding that launch's partial results where this launch keeps its counters)
      int* const tickets = reinterpret_cast<int*>(ws);
      unsigned char* const slots = ws + kPrefillTicketBytes;
      const int64_t bh = (int64_t)b * H + h;
      unsigned char* const base = slots + ((bh * (nqb - kPrefillChunkBlocks) + (qblock - kPrefillChunkBlocks)) * max_chunks) * (int64_t)PS::SLOT_BYTES;
      {
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(base + (int64_t)chunk * PS::SLOT_BYTES, PS::SLOT_BYTES);
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
#pragma unroll
          for (int ht = 0; ht < HT; ++ht)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, o[qt][ht]), rs, (((wave * QT + qt) * HT + ht) * 64 + lane) * 16, 0, 16 /* sc1 */);
          __builtin_amdgcn_raw_buffer_store_b64(u32x2{__float_as_uint(m[qt]), __float_as_uint(l[qt])}, rs,
                                                PS::O_BYTES + ((wave * QT + qt) * 64 + lane) * 8, 0, 16 /* sc1 */);
        }
      }
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));  // vmcnt(0): this wave's stores have landed
      __syncthreads();
      int* const s_last = reinterpret_cast<int*>(smem);  // the tiles are done with
      if (tid == 0) {
        int* tk = tickets + bh * nqb + qblock;
        const int t = __hip_atomic_fetch_add(tk, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *s_last = (t == nchunks - 1);
        if (t == nchunks - 1) __hip_atomic_store(tk, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
      }
      __syncthreads();
      if (!*s_last) return;
      // all runs in the order of their keys, this workgroup's own re-read like the others: which workgroup comes
      // last varies from launch to launch, the order of the additions must not
      for (int c = 0; c < nchunks; ++c) {
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(base + (int64_t)c * PS::SLOT_BYTES, PS::SLOT_BYTES);
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
          const u32x2 ml = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rs, PS::O_BYTES + ((wave * QT + qt) * 64 + lane) * 8, 0, 16));
          const float mo = __uint_as_float(ml.x), lo = __uint_as_float(ml.y);
          const float mn = c == 0 ? mo : fmaxf(m[qt], mo);
          const float a_acc = c == 0 ? 0.f : __builtin_amdgcn_exp2f(m[qt] - mn), a_new = __builtin_amdgcn_exp2f(mo - mn);
          l[qt] = c == 0 ? lo : l[qt] * a_acc + lo * a_new;
          m[qt] = mn;
#pragma unroll
          for (int ht = 0; ht < HT; ++ht) {
            const f32x4 oo = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, (((wave * QT + qt) * HT + ht) * 64 + lane) * 16, 0, 16));
#pragma unroll
            for (int r = 0; r < 4; ++r) o[qt][ht][r] = c == 0 ? oo[r] : o[qt][ht][r] * a_acc + oo[r] * a_new;
          }
        }
      }
    }
  }
  // ---- write O[q][hd]: lane holds hd = 16ht + 4kq + r for query col ------------------------------------------
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int t = q0 + qt * 16 + col;
    const float inv = 1.f / l[qt];
    if (t >= T) continue;
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
// decode: one query per (batch, head); keys split into chunks of 128, 192 or 256 (32, 48 or 64 per wave)
// =====================================================================================================
// A lane owns 8 channels of one key: LPK = HD/8 lanes cover a key row with one 16-byte load each,
// a wave covers 64/LPK keys per load instruction.  All K and V loads of the wave's keys are
// issued before the first use (the kernel is latency-bound at batch 1); the dot product is reduced
// over the LPK lanes with DPP adds.
constexpr int kFlagMergeFromChunks = 24;  // chunks per head from which "choose" takes the flag form of the in-kernel merge
constexpr int kLLSpinLimit = 1 << 21;  // polls of the merging workgroup before it gives up (seconds)
constexpr int kDecodeMinChunk = 128;  // the smallest chunk: what the workspace is sized for

// Keys per wave of the decode kernels (a workgroup of four waves takes four times as many).  Measured, us per
// launch at 32 / 48 / 64 keys per wave (hd 128):
//   32 heads x 2049 keys  16.1 / 14.5 / 16.3   (64 makes 9 chunks, the last with one key, and 288 workgroups leave CUs idle)
//   16 heads x 2101 keys  13.6 / 11.6 / 11.9     32 heads x 1001 keys  11.7 / 11.0 / 11.5
//   16 heads x 1001 keys   9.6 /  9.9 / 10.5     32 heads x  301 keys   9.0 / 10.1 / 11.3
//   40 heads x 4091 keys  34.1 / 29.4 / 29.1     8 x 32 heads x 2049 keys  65.8 / 67.0 / 63.4
// (the kernels as they are now, 32 heads x 2101 keys in a cache of 2192: 40 / 48 / 56 keys per wave 13.0 / 12.6 / 14.2)
// So: the longest run of keys per workgroup that still leaves the launch with clearly more workgroups than CUs, and
// short runs for short contexts, where a workgroup's serial walk over its keys is most of the launch.
inline int decode_keys_per_wave(int B, int H, int n_keys_max) {
  const int64_t heads = (int64_t)B * H;
  if (heads * ((n_keys_max + 255) / 256) >= 320) return 64;
  if (n_keys_max >= 1536) return 48;
  return 32;
}

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

template <int DT, int HD, int KPW>
__global__ __launch_bounds__(256) void attn_decode_kernel(const void* __restrict__ q, const void* __restrict__ kc,
                                                          const void* __restrict__ vc,
                                                          const float* __restrict__ key_bias, float* __restrict__ ws,
                                                          int H, int Hkv, int Lmax, int past_len,
                                                          const int32_t* __restrict__ past_dev, int nchunks_max,
                                                          int bias_stride, const int32_t* __restrict__ beam_src,
                                                          int src_stride, int prompt_len, int beam) {
  constexpr int LPK = HD / 8;                        // lanes per key (8 channels each)
  constexpr int KPI = 64 / LPK;                      // keys per wave iteration
  constexpr int ITERS = KPW / KPI;                   // iterations per wave
  constexpr int kDecodeChunk = 4 * KPW, kDecodeKeysPerWave = KPW;
  constexpr int VW = DT == O355_F32 ? 2 : 1;         // 16-byte vectors per 8 channels
  __shared__ float red_o[4][HD];
  __shared__ float red_ml[4][2];
  const int chunk = blockIdx.x, h = blockIdx.y, b = blockIdx.z, hk = h / (H / Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = lane % LPK, kslot = lane / LPK;
  const float scale = 1.f / sqrtf((float)HD);
  const float lowest = Act<DT>::lowest();
  const int64_t cbase = ((int64_t)b * Hkv + hk) * Lmax * HD;
  const int kbase = chunk * kDecodeChunk + wave * kDecodeKeysPerWave;
  const int kmax = min(nchunks_max * kDecodeChunk, Lmax) - 1;  // last row the launch may touch

  // ---- every load of this wave, issued up front.  The addresses do not depend on the position (it
  // may live in device memory and would cost a round trip first): rows past the end are clamped to
  // the launch bound, may be unwritten, and are discarded below. ----------------------------------
  u32x4 kreg[ITERS][VW], vreg[ITERS][VW];
  float bias[ITERS];
  // Beam search (beam_src given): row b is beam b % beam of sequence b / beam.  Its prompt rows are those of
  // the sequence's first beam; the row of its i-th generated token lives in cache row beam_src[b][i] (where
  // the beam that produced that token wrote it), so choosing parents moves table entries, not cache rows
  // (olmo/beam_search.py:1062-1078 gathers every cache tensor instead).
  int64_t kb[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int keyc = min(kbase + it * KPI + kslot, kmax);
    int64_t cb = cbase;
    if (beam_src) {
      int slot = (b / beam) * beam;
      if (keyc >= prompt_len) slot = beam_src[(int64_t)b * src_stride + min(keyc - prompt_len, src_stride - 1)];
      slot = min(max(slot, 0), (int)gridDim.z - 1);
      cb = ((int64_t)slot * Hkv + hk) * Lmax * HD;
    }
    kb[it] = cb + (int64_t)keyc * HD + sub * 8;
  }
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int64_t e = kb[it];
#pragma unroll
    for (int v = 0; v < VW; ++v) kreg[it][v] = reinterpret_cast<const u32x4*>(kc)[e * VW / 8 + v];
  }
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int keyc = min(kbase + it * KPI + kslot, kmax);
    const int64_t e = kb[it];
#pragma unroll
    for (int v = 0; v < VW; ++v) vreg[it][v] = reinterpret_cast<const u32x4*>(vc)[e * VW / 8 + v];
    // a row of key_bias holds bias_stride entries, which may be fewer than the rows the launch may touch
    // (eager steps pass exactly past_len + 1): keys past the end of the row are past L and discarded below
    bias[it] = key_bias ? key_bias[(int64_t)b * bias_stride + min(keyc, bias_stride - 1)] : 0.f;
  }
  float qr[8];
  Vec8<DT>::ld(q, ((int64_t)b * H + h) * HD + sub * 8, qr);
  const int L = (past_dev ? *past_dev : past_len) + 1;
  if (chunk * kDecodeChunk >= L) return;
#pragma unroll
  for (int it = 0; it < ITERS; ++it)
    if (kbase + it * KPI + kslot >= L) {
#pragma unroll
      for (int v = 0; v < VW; ++v) vreg[it][v] = u32x4{0u, 0u, 0u, 0u};  // unwritten rows: 0 * NaN
    }

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
  if constexpr (LPK <= 4) wmax = combine_xor<4>(wmax, MaxOp{});
  if constexpr (LPK <= 8) wmax = combine_xor<8>(wmax, MaxOp{});
  wmax = combine_xor<32>(combine_xor<16>(wmax, MaxOp{}), MaxOp{});
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
    auto over_slots = [](float v) {
      if constexpr (LPK <= 4) v = combine_xor<4>(v, AddOp{});
      if constexpr (LPK <= 8) v = combine_xor<8>(v, AddOp{});
      return combine_xor<32>(combine_xor<16>(v, AddOp{}), AddOp{});
    };
    lsum = over_slots(lsum);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = over_slots(acc[i]);
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
                                                                 int nchunks_max, int chunk_keys) {
  constexpr int UN = 32;  // partials fetched per round, every load before the first use
  const int h = blockIdx.x, b = blockIdx.y;
  const float* src = ws + ((int64_t)b * H + h) * nchunks_max * (HD + 2);
  float mm = -INFINITY, ov = 0.f, lv = 0.f;
  int nch = nchunks_max;  // refined once the position has arrived (slots past it hold stale values)
  for (int c0 = 0; c0 < nch; c0 += UN) {
    float m[UN], l[UN], o[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      if (c0 + u < nchunks_max) {  // uniform over the workgroup
        const float* p = src + (c0 + u) * (HD + 2);
        m[u] = p[HD], l[u] = p[HD + 1], o[u] = p[threadIdx.x];
      }
    }
    if (c0 == 0) {
      const int L = (past_dev ? *past_dev : past_len) + 1;
      nch = min((L + chunk_keys - 1) / chunk_keys, nchunks_max);
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

// ---- decode with the attention input folded in (bf16): QK-norm + rotary + cache append + attention ----
// qkv [B, (H+2*Hkv)*HD] is the fused projection of the one new token per sequence.  Every workgroup
// (chunk, head, batch) recomputes the two full-width sums of squares (olmo/model.py:603-605) from the
// 2*(H+Hkv)*HD bytes of q and k while its K/V loads are in flight, rotates its own head's q
// (olmo/model.py:298-324) into LDS, and the workgroup whose chunk holds the new position also forms
// the new key / value row, appends it to the cache (olmo/model.py:615-620) and uses it from LDS.
//
// RELAY: the launch is one leg of the two-stream decode relay (relay.hip).  qkv then holds tagged words (bf16 bits
// << 16 | epoch & 0xffff), qk_ssq tagged sums (float, low 4 bits = epoch & 0xf) and `out` receives tagged words; the cache rows -- which
// depend on no other launch of the step -- are requested first, and the few threads that read the token's q | k | v
// pieces and the sums of squares ask for them until every tag shows this step's epoch (at most spin_limit times).
template <int HD, int QV, int KPW, bool RELAY = false>  // QV: 16-byte pieces of the q (k) row per thread, H*HD/8 <= QV*256; KPW: keys per wave
__global__ __launch_bounds__(256) void attn_decode_fused_kernel(
    const uint16_t* __restrict__ qkv, const uint16_t* __restrict__ qw, const uint16_t* __restrict__ kw,
    const float* __restrict__ sin_t, const float* __restrict__ cos_t, uint16_t* __restrict__ kc,
    uint16_t* __restrict__ vc, const float* __restrict__ key_bias, float* __restrict__ ws, int H, int Hkv, int Lmax,
    int n_pos, int past_len, const int32_t* __restrict__ past_dev, int nchunks_max, int bias_stride, float eps,
    const float* __restrict__ qk_ssq, const float* __restrict__ rope_now, uint16_t* __restrict__ out,
    int* __restrict__ tickets, int ll, const int32_t* __restrict__ epoch_p = nullptr, int32_t* __restrict__ status = nullptr,
    int spin_limit = 0, const int32_t* __restrict__ hint_in = nullptr, int32_t* __restrict__ hint_out = nullptr) {
  constexpr int LPK = HD / 8, KPI = 64 / LPK, ITERS = KPW / KPI;
  constexpr int kDecodeChunk = 4 * KPW, kDecodeKeysPerWave = KPW;
  constexpr int HALF = HD / 2, CPH = HD / 16;  // pair chunks per head
  constexpr int ROWS = 4 * KPI;                 // partial results of the workgroup: one per (wave, key slot)
  __shared__ __align__(16) float red_o[ROWS][HD];
  __shared__ float red_ml[ROWS][2];
  __shared__ float red2[2][4];
  __shared__ __align__(16) float qs[HD];
  __shared__ __align__(16) u32x4 knew[HD / 8], vnew[HD / 8];
  __shared__ int s_last;
  __shared__ uint32_t s_flag;
  // Every argument at once: fetched where each is first used they come in seven batches, each a round trip of the
  // scalar cache to memory that the wave waits out.
  if constexpr (!RELAY)
    asm volatile("" ::"s"(qkv), "s"(qw), "s"(kw), "s"(sin_t), "s"(cos_t), "s"(kc), "s"(vc), "s"(key_bias), "s"(ws), "s"(H), "s"(Hkv),
                 "s"(Lmax), "s"(n_pos), "s"(past_len), "s"(past_dev), "s"(nchunks_max), "s"(bias_stride), "s"(eps), "s"(qk_ssq),
                 "s"(rope_now), "s"(out), "s"(tickets), "s"(ll));
  const int chunk = blockIdx.x, h = blockIdx.y, b = blockIdx.z, gsz = H / Hkv, hk = h / gsz;
  const int tid = threadIdx.x, lane = tid & 63;
  // ll (flags in the data): the workgroup of the head's last chunk merges.  Workgroups start in the order of their
  // index (chunks of a head are consecutive), so when it runs all the others of its head have started, and since
  // none of them ever waits they will finish; should that order ever not hold, its polling is bounded.  Every
  // workgroup reads the launch counter of the head first, before any other request, so that waiting for it later
  // waits for nothing else.  (Drawing a number per workgroup instead was measured: 17 device-scope read-modify-writes
  // on one address take 6 us to drain.)
  int my_epoch = 0;
  if (ll && tid == 0)
    my_epoch = __hip_atomic_load(tickets + (gridDim.z + b) * H + h, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int sub = lane % LPK, kslot = lane / LPK;
  const float scale = 1.f / sqrtf((float)HD);
  const float lowest = -3.3895313892515355e38f;
  const int64_t cbase = ((int64_t)b * Hkv + hk) * Lmax * HD;
  const int kbase = chunk * kDecodeChunk + wave * kDecodeKeysPerWave;
  const int kmax = min(nchunks_max * kDecodeChunk, Lmax) - 1;  // last row the launch may touch
  const int dq = H * HD, dk = Hkv * HD;
  const uint16_t* row = qkv + (int64_t)b * (dq + 2 * dk);
  const bool norm = (qw != nullptr);

  // ---- 0. the position.  Read from device memory (graph replay) it arrives late: every request issued
  // after the cache rows below queues behind 30+ MB of them.  So nothing on the way to the rotated query
  // may depend on it: the rotary rows of the current position are then taken from rope_now ([sin | cos],
  // refreshed once per decode step by olmo355_rope_advance) rather than looked up by position, and the
  // position itself is first needed for masking, long after it has arrived.
  // It is asked for as a vector request (an offset the compiler cannot see to be uniform): as a scalar one it would
  // hold up every later wait for a scalar, the scalar counter having no order.
  int pos_v = past_len;
  if (past_dev) {
    int zero_v = 0;
    asm volatile("" : "+v"(zero_v));
    pos_v = __builtin_amdgcn_raw_buffer_load_b32(make_rsrc(past_dev, 4), zero_v, 0, 0);
  }

  // ---- 1. this head's q / new-k pieces, norm weights, rotary rows, sums of squares; then the cache rows
  // of this wave.  Cache rows come through a buffer resource with a scalar offset per request and the
  // lane index as address (a wave's 64 pieces are contiguous).  Requests stay inside the cache by
  // construction, not by the resource's range check (what it does with a scalar offset beyond the range is
  // not relied on): one that would start past the last row the launch may touch is moved back onto the last
  // KPI rows; such rows, like every row at or past the new position, are discarded below (the new one is
  // replaced from LDS).
  // roles: threads [0,CPH) rotate q of head h; [32,32+CPH) the new key of head hk; [64,64+HD/8) copy v
  const bool role_q = tid < CPH, role_k = tid >= 32 && tid < 32 + CPH, role_v = tid >= 64 && tid < 64 + HD / 8;
  const int c = role_q ? tid : tid - 32, j = c * 8;
  u32x4 x1, x2, w1, w2, vrow;
  f32x4 cs1[2], cs2[2], sn1[2], sn2[2];
  if (role_q || role_k) {
    if constexpr (!RELAY) {
      const uint16_t* src = role_q ? row + h * HD : row + dq + hk * HD;
      x1 = reinterpret_cast<const u32x4*>(src + j)[0];
      x2 = reinterpret_cast<const u32x4*>(src + j + HALF)[0];
    }
    if (norm) {
      const uint16_t* wsrc = role_q ? qw + h * HD : kw + hk * HD;
      w1 = reinterpret_cast<const u32x4*>(wsrc + j)[0];
      w2 = reinterpret_cast<const u32x4*>(wsrc + j + HALF)[0];
    }
    const int pos_r = rope_now ? 0 : min(__builtin_amdgcn_readfirstlane(pos_v), n_pos - 1);  // (waits for it: the path without rope_now)
    const float* sp = rope_now ? rope_now : sin_t + (int64_t)pos_r * HD;
    const float* cp = rope_now ? rope_now + HD : cos_t + (int64_t)pos_r * HD;
#pragma unroll
    for (int v4 = 0; v4 < 2; ++v4) {
      cs1[v4] = reinterpret_cast<const f32x4*>(cp + j)[v4], cs2[v4] = reinterpret_cast<const f32x4*>(cp + j + HALF)[v4];
      sn1[v4] = reinterpret_cast<const f32x4*>(sp + j)[v4], sn2[v4] = reinterpret_cast<const f32x4*>(sp + j + HALF)[v4];
    }
  }
  if constexpr (!RELAY) {
    if (role_v) vrow = reinterpret_cast<const u32x4*>(row + dq + dk + hk * HD)[tid - 64];
  }
  float sq = 0.f, sk = 0.f;
  u32x4 qrow[QV], krow[QV];
  f32x4 ssq_q[2], ssq_k[2];  // added up where the scale factors are formed, after the cache rows have been asked for
  if (norm && !RELAY) {
    if (qk_ssq) {
      // per-tile partials left by the projection: wave 0 alone adds them up.  At most 512 per row (H * HD <= 8192):
      // two 16-byte requests per lane and row, all four on their way at once (a loop of single loads is a chain of
      // round trips to L2 ahead of the cache rows: 8 us per launch at batch 8), zeros past the row's end
      if (wave == 0) {
        const float* pr = qk_ssq + (int64_t)b * ((dq + 2 * dk) >> 4);
        const __amdgpu_buffer_rsrc_t rpq = make_rsrc(pr, (int64_t)(dq >> 4) * 4), rpk = make_rsrc(pr + (dq >> 4), (int64_t)(dk >> 4) * 4);
        ssq_q[0] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rpq, lane * 16, 0, 0));
        ssq_q[1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rpq, lane * 16 + 1024, 0, 0));
        ssq_k[0] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rpk, lane * 16, 0, 0));
        ssq_k[1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rpk, lane * 16 + 1024, 0, 0));
      }
    } else {
#pragma unroll
      for (int i = 0; i < QV; ++i) {
        const int idx = tid + i * 256;
        if (idx < (dq >> 3)) qrow[i] = reinterpret_cast<const u32x4*>(row)[idx];
        if (idx < (dk >> 3)) krow[i] = reinterpret_cast<const u32x4*>(row + dq)[idx];
      }
    }
  }
  // ---- relay: the token's pieces and the sums of squares are tagged; they are asked for once here, BEFORE the cache
  // rows (when the projection is done already they arrive first and the query is ready while the rows travel) ...
  uint32_t tag16 = 0, epoch = 0;
  const int relay_width = dq + 2 * dk;
  const __amdgpu_buffer_rsrc_t rt = make_rsrc(RELAY ? reinterpret_cast<const uint32_t*>(qkv) + (int64_t)b * relay_width : nullptr,
                                              RELAY ? (int64_t)relay_width * 4 : 0);
  const __amdgpu_buffer_rsrc_t rs2 = make_rsrc(RELAY && qk_ssq ? reinterpret_cast<const uint32_t*>(qk_ssq) + (int64_t)b * (relay_width >> 4) : nullptr,
                                               RELAY && qk_ssq ? (int64_t)(relay_width >> 4) * 4 : 0);
  const int relay_first = role_q ? h * HD + j : (role_k ? dq + hk * HD + j : dq + dk + hk * HD + (tid - 64) * 8);  // element
  const bool role = role_q || role_k || role_v;
  const int nq_p = dq >> 4, nk_p = dk >> 4;  // tagged sums of the q and the k part (float, low 4 bits = epoch & 0xf)
  u32x4 t[4], pq[2], pk[2];
  // workgroups whose chunk lies past the current length (a captured launch covers the cache's capacity) leave below
  // without having waited for anything
  const bool relay_work = RELAY && (chunk * kDecodeChunk < __builtin_amdgcn_readfirstlane(pos_v) + 1 || (ll && chunk == nchunks_max - 1));
  // (every request goes past the L2 -- device-coherent -- so that no poll finds a line there that was fetched before
  // the projection's stores)
  auto relay_ask = [&]() {
    auto ld = [&](__amdgpu_buffer_rsrc_t r, int voff, int soff) {
      return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 16));
    };
    if (role) {
      t[0] = ld(rt, relay_first * 4, 0);
      t[1] = ld(rt, relay_first * 4 + 16, 0);
      if (!role_v) {
        t[2] = ld(rt, (relay_first + HALF) * 4, 0);
        t[3] = ld(rt, (relay_first + HALF) * 4 + 16, 0);
      }
    }
    if (wave == 0 && norm) {
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        if (r * 256 < nq_p) pq[r] = ld(rs2, lane * 16, r * 1024);
        if (r * 256 < nk_p) pk[r] = ld(rs2, lane * 16, nq_p * 4 + r * 1024);
      }
    }
  };
  if constexpr (RELAY) {
    epoch = (uint32_t)*epoch_p, tag16 = epoch & 0xffffu;
    if (wave < 2 && relay_work && !hint_in) relay_ask();  // beside a running producer (hint word given) the rows are rarely there yet
  }
  // first row of the last request that fits; 0 for a cache shorter than one request, whose lanes past the end
  // the range check then sees (the scalar offset is 0)
  const int rowcap = max(kmax + 1 - KPI, 0);
  const __amdgpu_buffer_rsrc_t rk = make_rsrc(kc + cbase, (int64_t)(kmax + 1) * HD * 2);
  const __amdgpu_buffer_rsrc_t rv = make_rsrc(vc + cbase, (int64_t)(kmax + 1) * HD * 2);
  u32x4 kreg[ITERS], vreg[ITERS];
  float bias[ITERS];
  // cache rows are read once per step: non-temporal (aux bit 1), 0.5 us less per launch at context 2048
#pragma unroll
  for (int it = 0; it < ITERS; ++it)
    kreg[it] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rk, lane * 16, min(kbase + it * KPI, rowcap) * HD * 2, 2));
  // The value rows are asked for further down, once the query is in LDS: a CU takes a wave's requests only as fast
  // as earlier ones come back (24 of them occupy a wave for 2 to 3 us, measured with time stamps), and a wave that
  // is issuing them cannot look at the token's pieces when they arrive.  With the key rows alone ahead of it the
  // query is ready 1 us earlier and the scores of the first keys are formed while the value rows travel.
  auto ask_v = [&](int it) {
    vreg[it] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rv, lane * 16, min(kbase + it * KPI, rowcap) * HD * 2, 2));
    bias[it] = key_bias ? key_bias[(int64_t)b * bias_stride + min(min(kbase + it * KPI + kslot, kmax), bias_stride - 1)] : 0.f;  // keys past the row's end are past L
  };
  if constexpr (RELAY) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) ask_v(it);
  }

  if constexpr (RELAY) {
    // ---- 1'. ... and until they do, asked for again: these requests queue behind the cache rows, which have to
    // arrive anyway
    if (wave < 2 && relay_work) {
      bool gave_up = false, watched = false;
      for (int spins = 0;; ++spins) {
        bool ok = hint_in == nullptr || watched;  // nothing has been asked for before the hint was up
        if (wave == 0 && norm) {
#pragma unroll
          for (int r = 0; r < 2; ++r) {
            auto sok = [&](const u32x4& v) { return (((v.x ^ epoch) | (v.y ^ epoch) | (v.z ^ epoch) | (v.w ^ epoch)) & 0xfu) == 0u; };
            if (r * 256 + lane * 4 < nq_p) ok = ok && sok(pq[r]);
            if (r * 256 + lane * 4 < nk_p) ok = ok && sok(pk[r]);
          }
        }
        if (role) {
          auto tok = [&](const u32x4& v) { return (((v.x ^ tag16) | (v.y ^ tag16) | (v.z ^ tag16) | (v.w ^ tag16)) & 0xffffu) == 0u; };
          ok = ok && tok(t[0]) && tok(t[1]);
          if (!role_v) ok = ok && tok(t[2]) && tok(t[3]);
        }
        if (__builtin_amdgcn_ballot_w64(!ok) == 0) break;
        if (spins >= spin_limit) {
          gave_up = true;
          break;
        }
        if (hint_in && !watched) {  // the projection is still at work: watch the word its last workgroup sets (a hint; the tags decide)
          const __amdgpu_buffer_rsrc_t rh = make_rsrc(hint_in, O355_RELAY_HINT_COPIES * O355_RELAY_HINT_STRIDE);
          const int copy = ((((int)blockIdx.y * (int)gridDim.x + (int)blockIdx.x) * 2 + wave) & (O355_RELAY_HINT_COPIES - 1)) * O355_RELAY_HINT_STRIDE;
          for (; spins < spin_limit; ++spins) {
            asm volatile("" ::: "memory");  // the request is made again in every iteration
            if ((uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rh, 0, copy, 16) == epoch) break;
            __builtin_amdgcn_s_sleep(16);
          }
          watched = true;
        } else {
          __builtin_amdgcn_s_sleep(4);
        }
        asm volatile("" ::: "memory");  // the requests are made again in every iteration
        relay_ask();
      }
      if (gave_up && lane == 0) {
        __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (status[4]) atomicOr(status + 5, 8), atomicAdd(status + 7, 1);
      }
      auto pack8 = [](const u32x4& a, const u32x4& c) {  // eight tagged words -> eight bf16
        return u32x4{(a.x >> 16) | (a.y & 0xffff0000u), (a.z >> 16) | (a.w & 0xffff0000u), (c.x >> 16) | (c.y & 0xffff0000u),
                     (c.z >> 16) | (c.w & 0xffff0000u)};
      };
      if (role_q || role_k) x1 = pack8(t[0], t[1]), x2 = pack8(t[2], t[3]);
      if (role_v) vrow = pack8(t[0], t[1]);
      if (wave == 0 && norm) {
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          auto sm = [](const u32x4& v) {
            return (__uint_as_float(v.x & 0xfffffff0u) + __uint_as_float(v.y & 0xfffffff0u)) +
                   (__uint_as_float(v.z & 0xfffffff0u) + __uint_as_float(v.w & 0xfffffff0u));
          };
          if (r * 256 + lane * 4 < nq_p) sq += sm(pq[r]);
          if (r * 256 + lane * 4 < nk_p) sk += sm(pk[r]);
        }
      }
    }
  }
  // ---- 2. QK-norm scale factors, rotary, the new cache row --------------------------------------------------
  float rq = 1.f, rk_ = 1.f;
  u32x4 pk1, pk2;
  if (norm) {
    if (qk_ssq) {
      if (wave == 0) {
        if constexpr (!RELAY) {
          sq = ((ssq_q[0][0] + ssq_q[0][1]) + (ssq_q[0][2] + ssq_q[0][3])) + ((ssq_q[1][0] + ssq_q[1][1]) + (ssq_q[1][2] + ssq_q[1][3]));
          sk = ((ssq_k[0][0] + ssq_k[0][1]) + (ssq_k[0][2] + ssq_k[0][3])) + ((ssq_k[1][0] + ssq_k[1][1]) + (ssq_k[1][2] + ssq_k[1][3]));
        }
        sq = wave_sum(sq), sk = wave_sum(sk);
        rq = 1.f / sqrtf(sq / (float)dq + eps);
        rk_ = 1.f / sqrtf(sk / (float)dk + eps);
      }
    } else {
#pragma unroll
      for (int i = 0; i < QV; ++i) {
        const int idx = tid + i * 256;
        float f[8];
        if (idx < (dq >> 3)) {
          Vec8<O355_BF16>::unpack(reinterpret_cast<const u32x4(&)[1]>(qrow[i]), f);
#pragma unroll
          for (int e = 0; e < 8; ++e) sq += f[e] * f[e];
        }
        if (idx < (dk >> 3)) {
          Vec8<O355_BF16>::unpack(reinterpret_cast<const u32x4(&)[1]>(krow[i]), f);
#pragma unroll
          for (int e = 0; e < 8; ++e) sk += f[e] * f[e];
        }
      }
      sq = wave_sum(sq), sk = wave_sum(sk);
      if (lane == 0) red2[0][wave] = sq, red2[1][wave] = sk;
      lds_barrier();
      rq = 1.f / sqrtf((red2[0][0] + red2[0][1] + red2[0][2] + red2[0][3]) / (float)dq + eps);
      rk_ = 1.f / sqrtf((red2[1][0] + red2[1][1] + red2[1][2] + red2[1][3]) / (float)dk + eps);
    }
  }
  if (role_q || role_k) {
    float a1[8], a2[8], ww1[8], ww2[8];
    Vec8<O355_BF16>::unpack(reinterpret_cast<const u32x4(&)[1]>(x1), a1);
    Vec8<O355_BF16>::unpack(reinterpret_cast<const u32x4(&)[1]>(x2), a2);
    if (norm) {
      Vec8<O355_BF16>::unpack(reinterpret_cast<const u32x4(&)[1]>(w1), ww1);
      Vec8<O355_BF16>::unpack(reinterpret_cast<const u32x4(&)[1]>(w2), ww2);
    }
    const float r = role_q ? rq : rk_;
    float o1[8], o2[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float u1 = a1[e], u2 = a2[e];
      if (norm) {
        u1 = round_bf16(ww1[e] * round_bf16(u1 * r));
        u2 = round_bf16(ww2[e] * round_bf16(u2 * r));
      }
      o1[e] = round_bf16(__fadd_rn(__fmul_rn(u1, cs1[e >> 2][e & 3]), __fmul_rn(-u2, sn1[e >> 2][e & 3])));
      o2[e] = round_bf16(__fadd_rn(__fmul_rn(u2, cs2[e >> 2][e & 3]), __fmul_rn(u1, sn2[e >> 2][e & 3])));
    }
    if (role_q) {
#pragma unroll
      for (int e = 0; e < 8; ++e) qs[j + e] = o1[e], qs[j + HALF + e] = o2[e];
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) pk1[e] = pack_bf16x2(o1[2 * e], o1[2 * e + 1]), pk2[e] = pack_bf16x2(o2[2 * e], o2[2 * e + 1]);
      knew[c] = pk1, knew[c + CPH] = pk2;
    }
  }
  if (role_v) vnew[tid - 64] = vrow;
  // ---- the position is needed from here on ----------------------------------------------------------------
  const int pos = __builtin_amdgcn_readfirstlane(pos_v);
  const int L = pos + 1;
  const bool bad_pos = pos >= Lmax || pos >= n_pos || pos > kmax;
  bool merger = false, active = chunk * kDecodeChunk < L;
  uint32_t flag = 0;  // what this launch writes next to every number of a partial: a NaN pattern no partial holds
  if (ll) {
    if (tid == 0) s_flag = 0x7FC00000u | ((uint32_t)(my_epoch + 1) & 0x3FFFFFu);
    __syncthreads();
    merger = chunk == nchunks_max - 1, flag = s_flag;
    if (bad_pos || (!active && !merger)) return;  // an unusable position: nothing is computed, nothing to tidy up
  } else if (!active || bad_pos) {
    return;  // whole workgroup
  }
  if (pos / kDecodeChunk == chunk && h % gsz == 0) {  // the chunk that holds the new position appends it
    if (role_k) {
      const int64_t o = cbase + (int64_t)pos * HD + j;
      reinterpret_cast<u32x4*>(kc)[o >> 3] = pk1;
      reinterpret_cast<u32x4*>(kc)[(o + HALF) >> 3] = pk2;
    }
    if (role_v) reinterpret_cast<u32x4*>(vc)[(cbase + (int64_t)pos * HD + (tid - 64) * 8) >> 3] = vrow;
  }
  lds_barrier();
  float qr[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) qr[i] = qs[sub * 8 + i];
  if constexpr (!RELAY) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) ask_v(it);
  }

  // ---- 3. scores, softmax partial and P.V per key slot (the LPK lanes that share a key) ------------
  float s[ITERS];
  float smax = -INFINITY;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int key = kbase + it * KPI + kslot;
    if (key == pos) kreg[it] = knew[sub], vreg[it] = vnew[sub];
    if (key >= L) vreg[it] = u32x4{0u, 0u, 0u, 0u};  // unwritten rows: 0 * NaN
    float kf[8];
    Vec8<O355_BF16>::unpack(reinterpret_cast<const u32x4(&)[1]>(kreg[it]), kf);
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) d = __builtin_fmaf(qr[i], kf[i], d);
    d = group_sum<LPK>(d);
    float v = bias[it] <= kMaskThreshold ? lowest : d * scale + bias[it];
    v = key < L ? v : -INFINITY;
    s[it] = v;
    smax = fmaxf(smax, v);
  }
  // a slot whose keys all lie beyond L contributes nothing
  const bool empty = (kbase + kslot >= L);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float lsum = 0.f;
  if (!empty) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const float pw = __expf(s[it] - smax);
      lsum += pw;
      float vf[8];
      Vec8<O355_BF16>::unpack(reinterpret_cast<const u32x4(&)[1]>(vreg[it]), vf);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(pw, vf[i], acc[i]);
    }
  }
  {
    const int rrow = wave * KPI + kslot;
    f32x4* ro = reinterpret_cast<f32x4*>(&red_o[rrow][sub * 8]);
    ro[0] = f32x4{acc[0], acc[1], acc[2], acc[3]};
    ro[1] = f32x4{acc[4], acc[5], acc[6], acc[7]};
    if (sub == 0) red_ml[rrow][0] = empty ? -INFINITY : smax, red_ml[rrow][1] = empty ? 0.f : lsum;
  }
  __syncthreads();
  float mm = red_ml[0][0];
#pragma unroll
  for (int w = 1; w < ROWS; ++w) mm = fmaxf(mm, red_ml[w][0]);
  float* dst = ws + (((int64_t)b * H + h) * nchunks_max + chunk) * (HD + 2);
  float ov = 0.f, lv = 0.f;
  if (tid < HD) {
#pragma unroll
    for (int w = 0; w < ROWS; ++w) ov += red_o[w][tid] * __expf(red_ml[w][0] - mm);
  }
  if (tid == 0) {
#pragma unroll
    for (int w = 0; w < ROWS; ++w) lv += red_ml[w][1] * __expf(red_ml[w][0] - mm);
  }
  if (!tickets) {  // partials merged by attn_decode_combine_kernel
    if (tid < HD) dst[tid] = ov;
    if (tid == 0) dst[HD] = mm, dst[HD + 1] = lv;
    return;
  }
  if (ll) {
    // ---- 4'. flags in the data.  A partial is (HD + 2) pairs (number, flag) written with 8-byte device-scope
    // stores, so a reader that sees this launch's flag sees the number too: the writers do not wait for their
    // stores, draw no second ticket and leave; the merging workgroup polls the pairs of the other chunks.
    const int nact = min((L + kDecodeChunk - 1) / kDecodeChunk, nchunks_max);
    uint64_t* w64 = reinterpret_cast<uint64_t*>(ws) + ((int64_t)b * H + h) * nchunks_max * (HD + 2);
    auto pair_of = [&](float v) { return (uint64_t)__float_as_uint(v) | ((uint64_t)flag << 32); };
    if (!merger) {
      uint64_t* d64 = w64 + (int64_t)chunk * (HD + 2);
      if (tid < HD) __hip_atomic_store(d64 + tid, pair_of(ov), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (tid == 0) {
        __hip_atomic_store(d64 + HD, pair_of(mm), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(d64 + HD + 1, pair_of(lv), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      return;
    }
    if (tid == 0) red2[0][0] = mm, red2[0][1] = lv;  // this workgroup's own share stays on chip
    __syncthreads();
    if (tid >= HD) return;
    float gm = active ? red2[0][0] : -INFINITY, go = active ? ov : 0.f, gl = active ? red2[0][1] : 0.f;
    constexpr int UN = 8;
    bool gave_up = false;
    for (int c0 = 0; c0 < nact; c0 += UN) {
      uint64_t po[UN], pm[UN], pl[UN];
      for (int spins = 0;; ++spins) {
        bool ok = true;
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          const int c = c0 + u;
          if (c < nact && !(active && c == chunk)) {
            const uint64_t* pp = w64 + (int64_t)c * (HD + 2);
            po[u] = __hip_atomic_load(pp + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            pm[u] = __hip_atomic_load(pp + HD, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            pl[u] = __hip_atomic_load(pp + HD + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          const int c = c0 + u;
          if (c < nact && !(active && c == chunk))
            ok = ok && (uint32_t)(po[u] >> 32) == flag && (uint32_t)(pm[u] >> 32) == flag && (uint32_t)(pl[u] >> 32) == flag;
        }
        if (ok) break;
        if (spins > kLLSpinLimit) { gave_up = true; break; }  // never seen: a writer that died; the result is marked
        __builtin_amdgcn_s_sleep(1);
      }
      float rm = gm;
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int c = c0 + u;
        if (c < nact && !(active && c == chunk)) rm = fmaxf(rm, __uint_as_float((uint32_t)pm[u]));
      }
      const float a = __expf(gm - rm);  // exp(-inf) = 0 while nothing has been merged yet
      go *= a, gl *= a;
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int c = c0 + u;
        if (c < nact && !(active && c == chunk)) {
          const float wgt = __expf(__uint_as_float((uint32_t)pm[u]) - rm);
          go += __uint_as_float((uint32_t)po[u]) * wgt, gl += __uint_as_float((uint32_t)pl[u]) * wgt;
        }
      }
      gm = rm;
    }
    {
      const uint16_t bits = gave_up ? (uint16_t)0x7FC0 : f32_to_bf16_bits(go / gl);
      if constexpr (RELAY)
        __hip_atomic_store(reinterpret_cast<uint32_t*>(out) + ((int64_t)b * H + h) * HD + tid, ((uint32_t)bits << 16) | tag16,
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else out[((int64_t)b * H + h) * HD + tid] = bits;
    }
    if (RELAY && hint_out && tid < O355_RELAY_HINT_COPIES && h == H - 1 && b == (int)gridDim.z - 1)
      __hip_atomic_store(hint_out + tid * (O355_RELAY_HINT_STRIDE / 4), (int32_t)epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0)  // the next launch's flag
      __hip_atomic_store(tickets + (gridDim.z + b) * H + h, (int)(flag & 0x3FFFFFu), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;
  }
  // ---- 4. the last workgroup of a (batch, head) to finish merges the partials itself ---------------------
  // Partials are published with device-scope stores (they bypass the per-XCD L2), each wave waits
  // until its stores are acknowledged, then one thread takes a ticket with a device-scope atomic;
  // whoever draws the last ticket reads all partials back with device-scope loads.  No workgroup
  // ever waits for another one.
  if (tid < HD) __hip_atomic_store(dst + tid, ov, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (tid == 0) {
    __hip_atomic_store(dst + HD, mm, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(dst + HD + 1, lv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));  // vmcnt(0): this wave's stores have landed
  __syncthreads();
  const int nact = min((L + kDecodeChunk - 1) / kDecodeChunk, nchunks_max);
  if (tid == 0) {
    int* tk = tickets + b * H + h;
    const int t = __hip_atomic_fetch_add(tk, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (t == nact - 1);
    if (t == nact - 1) __hip_atomic_store(tk, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
  }
  __syncthreads();
  if (!s_last || tid >= HD) return;
  const float* src = ws + ((int64_t)b * H + h) * nchunks_max * (HD + 2);
  constexpr int UN = 16;
  float gm = -INFINITY, go = 0.f, gl = 0.f;
  for (int c0 = 0; c0 < nact; c0 += UN) {
    float m[UN], l[UN], o[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u)
      if (c0 + u < nact) {
        const float* pp = src + (c0 + u) * (HD + 2);
        m[u] = __hip_atomic_load(pp + HD, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        l[u] = __hip_atomic_load(pp + HD + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        o[u] = __hip_atomic_load(pp + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    float rm = gm;
#pragma unroll
    for (int u = 0; u < UN; ++u)
      if (c0 + u < nact) rm = fmaxf(rm, m[u]);
    const float a = __expf(gm - rm);  // exp(-inf) = 0 on the first round
    go *= a, gl *= a;
#pragma unroll
    for (int u = 0; u < UN; ++u)
      if (c0 + u < nact) {
        const float wgt = __expf(m[u] - rm);
        go += o[u] * wgt, gl += l[u] * wgt;
      }
    gm = rm;
  }
  if constexpr (RELAY)
    __hip_atomic_store(reinterpret_cast<uint32_t*>(out) + ((int64_t)b * H + h) * HD + tid,
                       ((uint32_t)f32_to_bf16_bits(go / gl) << 16) | tag16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else out[((int64_t)b * H + h) * HD + tid] = f32_to_bf16_bits(go / gl);
  if (RELAY && hint_out && tid < O355_RELAY_HINT_COPIES && h == H - 1 && b == (int)gridDim.z - 1)
    __hip_atomic_store(hint_out + tid * (O355_RELAY_HINT_STRIDE / 4), (int32_t)epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int DT, int HD>
int launch_decode(const void* q, const void* kc, const void* vc, const float* key_bias, void* out, float* ws, int B,
                  int H, int Hkv, int Lmax, int past_len, const int32_t* past_dev, int n_keys_max, int bias_stride,
                  const int32_t* beam_src, int src_stride, int prompt_len, int beam, hipStream_t stream) {
  const int kpw = decode_keys_per_wave(B, H, n_keys_max), chunk = 4 * kpw;
  const int nch = (n_keys_max + chunk - 1) / chunk;
#define DECODE(KPWv)                                                                                                  \
  hipLaunchKernelGGL((attn_decode_kernel<DT, HD, KPWv>), dim3(nch, H, B), dim3(256), 0, stream, q, kc, vc, key_bias, \
                     ws, H, Hkv, Lmax, past_len, past_dev, nch, bias_stride, beam_src, src_stride, prompt_len, beam)
  if (kpw == 64) DECODE(64);
  else if (kpw == 48) DECODE(48);
  else DECODE(32);
#undef DECODE
  hipLaunchKernelGGL((attn_decode_combine_kernel<DT, HD>), dim3(H, B), dim3(HD), 0, stream, ws, out, H, past_len,
                     past_dev, nch, chunk);
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

namespace {
// Query rows that see only masked keys.  The reference gives a masked score the dtype's most negative
// *finite* value -- padding keys and keys after the query alike (olmo/model.py:375-381,1337-1376,
// olmo/torch_util.py:81-90) -- so for such a row every key of the call, later ones included, has the
// same score and the softmax is uniform over all of them: the row's output is the plain mean of the
// values of all past_len + T keys.  The attention kernels skip later keys, so this pass rewrites those rows
// (positions before a sequence's first unmasked key: the padding positions of a left-padded batch).
// One workgroup per (kv head, sequence); sums in a fixed order.
template <int DT>
__global__ __launch_bounds__(256) void attn_masked_rows_kernel(const void* __restrict__ vc, const float* __restrict__ key_bias,
                                                               void* __restrict__ out, int T, int H, int Hkv, int hd,
                                                               int Lmax, int past_len, int bias_stride) {
  __shared__ int first;
  __shared__ float part[256];
  const int hk = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int L = past_len + T;
  if (tid == 0) first = L;
  __syncthreads();
  for (int k = tid; k < L; k += 256)
    if (key_bias[(int64_t)b * bias_stride + k] > kMaskThreshold) atomicMin(&first, k);
  __syncthreads();
  const int nrows = min(first, L) - past_len;  // query rows t < nrows sit before the first unmasked key
  if (nrows <= 0) return;                      // workgroup-uniform
  const int nsl = 256 / hd, c = tid % hd, sl = tid / hd;
  const int64_t vbase = ((int64_t)b * Hkv + hk) * Lmax * hd;
  float acc = 0.f;
  if (sl < nsl)
    for (int k = sl; k < L; k += nsl) acc += Act<DT>::ld(vc, vbase + (int64_t)k * hd + c);
  part[tid] = acc;
  __syncthreads();
  if (sl == 0) {
    float sum = 0.f;
    for (int j = 0; j < nsl; ++j) sum += part[j * hd + c];
    const float mean = sum / (float)L;
    const int rep = H / Hkv;
    for (int t = 0; t < nrows; ++t)
      for (int h = hk * rep; h < (hk + 1) * rep; ++h) Act<DT>::st(out, ((int64_t)(b * T + t) * H + h) * hd + c, mean);
  }
}

int attn_prefill_main(const void* q, const void* kcache, const void* vcache, const float* key_bias, void* out, int B, int T,
                      int H, int Hkv, int hd, int Lmax, int past_len, int bias_stride, int dtype, hipStream_t s, void* ws,
                      int64_t ws_bytes);
bool prefill_split_applies(int B, int T, int H, int hd, int past_len, int dtype);
int64_t prefill_split_bytes(int B, int T, int H, int hd);

int attn_prefill_any(const void* q, const void* kcache, const void* vcache, const float* key_bias, void* out, void* ws,
                     int64_t ws_bytes, int B, int T, int H, int Hkv, int hd, int Lmax, int past_len, int bias_stride, int dtype,
                     void* stream) {
  if (!q || !kcache || !vcache || !out) return O355_EINVAL;
  if (hd <= 0 || hd > 256) return O355_EUNSUPPORTED;
  hipStream_t s = as_stream(stream);
  const int rc = attn_prefill_main(q, kcache, vcache, key_bias, out, B, T, H, Hkv, hd, Lmax, past_len, bias_stride, dtype, s, ws, ws_bytes);
  if (rc != O355_OK || !key_bias) return rc;
  if (dtype == O355_BF16)
    hipLaunchKernelGGL(attn_masked_rows_kernel<O355_BF16>, dim3(Hkv, B), dim3(256), 0, s, vcache, key_bias, out, T, H, Hkv,
                       hd, Lmax, past_len, bias_stride);
  else if (dtype == O355_F16)
    hipLaunchKernelGGL(attn_masked_rows_kernel<O355_F16>, dim3(Hkv, B), dim3(256), 0, s, vcache, key_bias, out, T, H, Hkv,
                       hd, Lmax, past_len, bias_stride);
  else
    hipLaunchKernelGGL(attn_masked_rows_kernel<O355_F32>, dim3(Hkv, B), dim3(256), 0, s, vcache, key_bias, out, T, H, Hkv,
                       hd, Lmax, past_len, bias_stride);
  O355_CHECK_LAUNCH();
}
}  // namespace

extern "C" int olmo355_attn_prefill(const void* q, const void* kcache, const void* vcache, const float* key_bias,
                                    void* out, int B, int T, int H, int Hkv, int hd, int Lmax, int past_len,
                                    int bias_stride, int dtype, void* stream) {
  return attn_prefill_any(q, kcache, vcache, key_bias, out, nullptr, 0, B, T, H, Hkv, hd, Lmax, past_len, bias_stride, dtype, stream);
}

// olmo355_attn_prefill with a workspace: where olmo355_attn_prefill_workspace_bytes(...) is not 0 the launch shares the
// long query blocks between workgroups along the keys (see attn_prefill_mfma_kernel) and needs that many bytes, zeroed
// when allocated (it starts with one int32 counter per (batch, head, query block), which every launch leaves at zero
// again); O355_EINVAL when ws_bytes is smaller.  ws == NULL or a size of 0: the plain launch.
extern "C" int64_t olmo355_attn_prefill_workspace_bytes(int B, int T, int H, int hd, int past_len, int dtype) {
  if (B <= 0 || T <= 0 || H <= 0 || !prefill_split_applies(B, T, H, hd, past_len, dtype)) return 0;
  return prefill_split_bytes(B, T, H, hd);
}
extern "C" int olmo355_attn_prefill_ws(const void* q, const void* kcache, const void* vcache, const float* key_bias,
                                       void* out, void* ws, int64_t ws_bytes, int B, int T, int H, int Hkv, int hd, int Lmax,
                                       int past_len, int bias_stride, int dtype, void* stream) {
  return attn_prefill_any(q, kcache, vcache, key_bias, out, ws, ws_bytes, B, T, H, Hkv, hd, Lmax, past_len, bias_stride, dtype, stream);
}

namespace {
// The key-split form pays when the plain launch is a single round of workgroups of very unequal length: a prompt from
// scratch (past_len == 0) with at most 1024 (batch, head, query block) triples.  The run length: 8 query blocks' worth
// of keys while the plain launch would leave places on the chip empty (two workgroups per CU), 12 once every place is
// taken (then only the few longest blocks are worth a hand-over).  Measured, 2048 tokens, us per launch, plain / runs
// of 8 / 10 / 12 / 14: 16 heads of 128 (256 triples) 52.6 / 37.7-39.5 / 40.7 / 45.4 / 49.9; 32 heads of 128 (512 triples)
// 61.4 / 65.6 / 61.0 / 56.8 / 60.6; 32 heads of 64 41.8 / - / 34.4 / 35.7 / 37.9.
int prefill_chunk_blocks(int B, int T, int H) {
  const int nqb = (T + 127) / 128;
  return (int64_t)B * H * nqb <= 384 ? 8 : 12;
}
bool prefill_split_applies(int B, int T, int H, int hd, int past_len, int dtype) {
  const int nqb = (T + 127) / 128, cb = prefill_chunk_blocks(B, T, H);
  return dtype == O355_BF16 && (hd == 128 || hd == 64) && past_len == 0 && nqb > cb && nqb <= cb * kPrefillMaxChunks &&
         (int64_t)B * H * nqb <= kPrefillMaxTriples;
}
int64_t prefill_split_bytes(int B, int T, int H, int hd) {
  const int nqb = (T + 127) / 128, cb = prefill_chunk_blocks(B, T, H), maxc = (nqb - 1) / cb + 1;
  static_assert(kPrefillMaxTriples * 4 <= kPrefillTicketBytes, "one counter per triple");
  const int64_t slot = hd == 128 ? PrefillSplit<128>::SLOT_BYTES : PrefillSplit<64>::SLOT_BYTES;
  return kPrefillTicketBytes + (int64_t)B * H * (nqb - cb) * maxc * slot;
}

int attn_prefill_main(const void* q, const void* kcache, const void* vcache, const float* key_bias, void* out, int B, int T,
                      int H, int Hkv, int hd, int Lmax, int past_len, int bias_stride, int dtype, hipStream_t s, void* ws,
                      int64_t ws_bytes) {
  if (B <= 0 || T <= 0 || H <= 0 || Hkv <= 0 || H % Hkv || past_len < 0 || past_len + T > Lmax) return O355_EINVAL;
  if (key_bias && bias_stride < past_len + T) return O355_EINVAL;
  if (dtype == O355_BF16 && (hd == 128 || hd == 64) && (int64_t)Lmax * hd < (1ll << 31)) {  // 32-bit offsets within a head
    const int nqb = (T + 127) / 128;
    if (ws && prefill_split_applies(B, T, H, hd, past_len, dtype)) {
      if (ws_bytes < prefill_split_bytes(B, T, H, hd)) return O355_EINVAL;
      const int cb = prefill_chunk_blocks(B, T, H);
      int n_wg = 0;
      for (int b = 0; b < nqb; ++b) n_wg += b / cb + 1;
      const int maxc = (nqb - 1) / cb + 1;
      const dim3 grid(H, n_wg, B);  // heads fastest, then (block, run of keys) longest first (see the kernel)
      if (hd == 128) {
        constexpr int lds = PrefillLds<128>::BYTES;
        auto kern = attn_prefill_mfma_kernel<128>;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
          return O355_ELAUNCH;
        hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, (const uint16_t*)q, (const uint16_t*)kcache, (const uint16_t*)vcache,
                           key_bias, (uint16_t*)out, T, H, Hkv, Lmax, past_len, bias_stride, (unsigned char*)ws, maxc, cb);
      } else {
        hipLaunchKernelGGL(attn_prefill_mfma_kernel<64>, grid, dim3(256), PrefillLds<64>::BYTES, s, (const uint16_t*)q,
                           (const uint16_t*)kcache, (const uint16_t*)vcache, key_bias, (uint16_t*)out, T, H, Hkv, Lmax,
                           past_len, bias_stride, (unsigned char*)ws, maxc, cb);
      }
      O355_CHECK_LAUNCH();
    }
    const dim3 grid(H, nqb, B);  // heads fastest, then query blocks by rank (see the kernel)
    if (hd == 128) {
      constexpr int lds = PrefillLds<128>::BYTES;  // more than a launch gets without asking
      auto kern = attn_prefill_mfma_kernel<128>;
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
        return O355_ELAUNCH;
      hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, (const uint16_t*)q, (const uint16_t*)kcache,
                         (const uint16_t*)vcache, key_bias, (uint16_t*)out, T, H, Hkv, Lmax, past_len, bias_stride, nullptr, 1, 8);
    } else {
      hipLaunchKernelGGL(attn_prefill_mfma_kernel<64>, grid, dim3(256), PrefillLds<64>::BYTES, s, (const uint16_t*)q,
                         (const uint16_t*)kcache, (const uint16_t*)vcache, key_bias, (uint16_t*)out, T, H, Hkv, Lmax,
                         past_len, bias_stride, nullptr, 1, 8);
    }
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
  } else if (dtype == O355_F16) {
    if (hd == 32) GENERIC(O355_F16, 32);
    if (hd == 64) GENERIC(O355_F16, 64);
    if (hd == 128) GENERIC(O355_F16, 128);
  }
#undef GENERIC
  return O355_EUNSUPPORTED;
}
}  // namespace

namespace {
// *pos += delta, then rope_now = [sin_tab[*pos] | cos_tab[*pos]] (the last table row when *pos runs past it)
__global__ void rope_advance_kernel(int32_t* __restrict__ pos, int delta, const float* __restrict__ sin_t,
                                    const float* __restrict__ cos_t, float* __restrict__ rope_now, int hd, int n_pos) {
  const int p = *pos + delta;
  __syncthreads();  // every thread has read the old value
  if (threadIdx.x == 0) *pos = p;
  const int r = min(max(p, 0), n_pos - 1);
  for (int i = threadIdx.x; i < hd; i += blockDim.x) {
    rope_now[i] = sin_t[(int64_t)r * hd + i];
    rope_now[hd + i] = cos_t[(int64_t)r * hd + i];
  }
}
}  // namespace

extern "C" int olmo355_rope_advance(int32_t* pos, int delta, const float* sin_tab, const float* cos_tab, float* rope_now,
                                    int hd, int n_pos, void* stream) {
  if (!pos || !sin_tab || !cos_tab || !rope_now || hd <= 0 || n_pos <= 0) return O355_EINVAL;
  hipLaunchKernelGGL(rope_advance_kernel, dim3(1), dim3(128), 0, as_stream(stream), pos, delta, sin_tab, cos_tab, rope_now,
                     hd, n_pos);
  O355_CHECK_LAUNCH();
}

extern "C" int64_t olmo355_attn_decode_workspace_bytes(int B, int H, int hd, int n_keys_max) {
  if (B <= 0 || H <= 0 || hd <= 0 || n_keys_max <= 0) return 0;
  const int64_t nch = (n_keys_max + kDecodeMinChunk - 1) / kDecodeMinChunk;  // longer chunks need less
  // two counters per (batch, head), then the partials: (hd + 2) numbers per chunk, each with room for a flag word
  return (int64_t)B * H * 8 + (int64_t)B * H * nch * (hd + 2) * 8;
}

namespace {
int attn_decode_any(const void* q, const void* kcache, const void* vcache, const float* key_bias, void* out, void* ws,
                    int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax, int past_len, const int32_t* past_len_dev,
                    int n_keys_max, int bias_stride, const int32_t* beam_src, int src_stride, int prompt_len, int beam,
                    int dtype, void* stream) {
  if (!q || !kcache || !vcache || !out || !ws) return O355_EINVAL;
  if (B <= 0 || H <= 0 || Hkv <= 0 || H % Hkv || past_len < 0 || n_keys_max <= 0 || n_keys_max > Lmax)
    return O355_EINVAL;
  // the launch writes one partial per (sequence, head, chunk): the workspace must hold them all
  if (ws_bytes < olmo355_attn_decode_workspace_bytes(B, H, hd, n_keys_max)) return O355_EINVAL;
  if (!past_len_dev && past_len + 1 > n_keys_max) return O355_EINVAL;
  if (key_bias && bias_stride < n_keys_max) return O355_EINVAL;
  if (beam_src && (beam <= 0 || B % beam || prompt_len < 0 || src_stride <= 0 || prompt_len + src_stride < n_keys_max))
    return O355_EINVAL;
  hipStream_t s = as_stream(stream);
#define DECODE(DTv, HDv)                                                                                          \
  return launch_decode<DTv, HDv>(q, kcache, vcache, key_bias, out, (float*)ws + (int64_t)2 * B * H, B, H, Hkv, Lmax, past_len, \
                                 past_len_dev, n_keys_max, bias_stride, beam_src, src_stride, prompt_len, beam, s)
  if (dtype == O355_BF16) {
    if (hd == 128) DECODE(O355_BF16, 128);
    if (hd == 64) DECODE(O355_BF16, 64);
    if (hd == 32) DECODE(O355_BF16, 32);
  } else if (dtype == O355_F32) {
    if (hd == 128) DECODE(O355_F32, 128);
    if (hd == 64) DECODE(O355_F32, 64);
    if (hd == 32) DECODE(O355_F32, 32);
  } else if (dtype == O355_F16) {
    if (hd == 128) DECODE(O355_F16, 128);
    if (hd == 64) DECODE(O355_F16, 64);
    if (hd == 32) DECODE(O355_F16, 32);
  }
#undef DECODE
  return O355_EUNSUPPORTED;
}
}  // namespace

extern "C" int olmo355_attn_decode(const void* q, const void* kcache, const void* vcache, const float* key_bias,
                                   void* out, void* ws, int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax, int past_len,
                                   const int32_t* past_len_dev, int n_keys_max, int bias_stride, int dtype,
                                   void* stream) {
  return attn_decode_any(q, kcache, vcache, key_bias, out, ws, ws_bytes, B, H, Hkv, hd, Lmax, past_len, past_len_dev, n_keys_max,
                         bias_stride, nullptr, 0, 0, 1, dtype, stream);
}

extern "C" int olmo355_attn_decode_beam(const void* q, const void* kcache, const void* vcache, const float* key_bias,
                                        void* out, void* ws, int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax, int past_len,
                                        const int32_t* past_len_dev, int n_keys_max, int bias_stride,
                                        const int32_t* beam_src, int src_stride, int prompt_len, int beam, int dtype,
                                        void* stream) {
  if (!beam_src) return O355_EINVAL;
  return attn_decode_any(q, kcache, vcache, key_bias, out, ws, ws_bytes, B, H, Hkv, hd, Lmax, past_len, past_len_dev, n_keys_max,
                         bias_stride, beam_src, src_stride, prompt_len, beam, dtype, stream);
}

// ---- olmo355_attn_decode without a workspace argument and without any allocation ------------------------------
// For callers that cannot allocate (HIP graph capture, tight serving loops): the per-chunk partial results
// (o, max, sum) live in a file-scope device array instead of a caller-provided workspace.  Each GPU holds its own
// copy of the array at its own address, found once per device with hipGetSymbolAddress (the array's name is not a
// device address in host code).  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two
// streams, two host threads) race.  Nothing in it has to start at zero: every partial a launch's combine kernel
// reads was written by the same launch's first kernel.
namespace {
constexpr int64_t kStaticScratchBytes = 16ll << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
void* g_scratch_ptr[kMaxDevices];      // per device, set once under the mutex
bool g_scratch_known[kMaxDevices];
std::mutex g_scratch_mutex;

int scratch_of_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return O355_ELAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_known[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return O355_ELAUNCH;
    g_scratch_ptr[dev] = p;
    g_scratch_known[dev] = true;
  }
  *out = g_scratch_ptr[dev];
  return O355_OK;
}
}  // namespace

extern "C" int64_t olmo355_attn_decode_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int olmo355_attn_decode_static(const void* q, const void* kcache, const void* vcache, const float* key_bias,
                                          void* out, int B, int H, int Hkv, int hd, int Lmax, int past_len,
                                          const int32_t* past_len_dev, int n_keys_max, int bias_stride, int dtype,
                                          void* stream) {
  if (B <= 0 || H <= 0 || hd <= 0 || n_keys_max <= 0) return O355_EINVAL;
  if (olmo355_attn_decode_workspace_bytes(B, H, hd, n_keys_max) > kStaticScratchBytes) return O355_ETOOBIG;
  void* ws = nullptr;
  const int st = scratch_of_current_device(&ws);
  if (st != O355_OK) return st;
  return attn_decode_any(q, kcache, vcache, key_bias, out, ws, kStaticScratchBytes, B, H, Hkv, hd, Lmax, past_len, past_len_dev,
                         n_keys_max, bias_stride, nullptr, 0, 0, 1, dtype, stream);
}

// merge: how the key chunks of a (batch, head) are merged: -1 = choose, 0 = in the kernel by the workgroup that
// finishes last (a ticket drawn after its stores have landed), 1 = in the kernel by the workgroup of the head's last
// chunk, which polls flags stored with the numbers, 2 = the separate combine kernel
namespace {
struct FusedPlan {
  int kpw, nch, ll;
  bool merge_in_kernel;
};
FusedPlan fused_plan(int B, int H, int n_keys_max, int merge) {
  FusedPlan p;
  p.kpw = decode_keys_per_wave(B, H, n_keys_max);
  p.nch = (n_keys_max + 4 * p.kpw - 1) / (4 * p.kpw);
  // (measured at the 7B shapes, context 2048: the in-kernel merge wins while the launch is a single round of
  // workgroups -- 17.0 against 20.4 us at batch 1 -- and loses once workgroups queue up -- 69.7 against 61.6 us
  // at batch 8, where one workgroup per (batch, head) takes 66.9)
  // (measured again with the value rows asked for behind the query, batch 8 and more, 32 heads: the flag form
  // 51.7 / 93.2 / 92.3 / 176.2 us at 8 x 2049, 16 x 2049, 8 x 4097, 32 x 2049 keys against 52.8 / 95.3 / 95.1 / 181.9 for
  // the separate kernel and 54.4 / 102.5 / 103.1 / 193.2 for tickets -- when the workgroups fill whole rounds of the
  // CUs; at 8 x 40 heads, 11.25 rounds, the separate kernel stays ahead, 63.1 against 65.1)
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0, cus = 0;
    n_cu = hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0 ? cus : 256;
  }
  const int64_t wgs = (int64_t)B * H * p.nch;
  const bool whole_rounds = wgs > 1536 && wgs % n_cu == 0;
  p.merge_in_kernel = merge == 0 || merge == 1 || (merge < 0 && (wgs <= 1536 || whole_rounds));
  // (measured with 128-key chunks, batch 1: the flag form is level with the ticket form at 17 chunks per head -- 17.2
  // against 16.4 us, 7B at context 2048 -- and ahead from about two dozen -- 34.4 against 36.5 us, 13B at context 4090;
  // with that launch's 256-key chunks, 17 per head, the two forms are level again at 29.6 us)
  p.ll = p.merge_in_kernel && (merge == 1 || (merge < 0 && (p.nch >= kFlagMergeFromChunks || whole_rounds))) ? 1 : 0;  // needs the counters
  return p;
}

int attn_fused_any(const void* qkv, const void* qw, const void* kw, const float* sin_tab, const float* cos_tab, void* kcache,
                   void* vcache, const float* key_bias, void* out, void* ws, int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax,
                   int n_pos, int past_len, const int32_t* past_len_dev, int n_keys_max, int bias_stride, float eps, const void* qk_ssq,
                   const float* rope_now, int dtype, int merge, bool relay, const int32_t* epoch, int32_t* status, int spin_limit,
                   const int32_t* hint_in, int32_t* hint_out, void* stream) {
  if (merge < -1 || merge > 2) return O355_EINVAL;
  if (!qkv || !sin_tab || !cos_tab || !kcache || !vcache || !out || !ws) return O355_EINVAL;
  if (B <= 0 || H <= 0 || Hkv <= 0 || H % Hkv || past_len < 0 || n_keys_max <= 0 || n_keys_max > Lmax)
    return O355_EINVAL;
  if ((qw == nullptr) != (kw == nullptr)) return O355_EINVAL;
  if (ws_bytes < olmo355_attn_decode_workspace_bytes(B, H, hd, n_keys_max)) return O355_EINVAL;
  if (!past_len_dev && (past_len + 1 > n_keys_max || past_len + 1 > n_pos)) return O355_EINVAL;
  if (key_bias && bias_stride < n_keys_max) return O355_EINVAL;
  if (dtype != O355_BF16 || (hd != 128 && hd != 64) || H * hd > 8 * 4 * 256) return O355_EUNSUPPORTED;
  hipStream_t s = as_stream(stream);
  const FusedPlan plan = fused_plan(B, H, n_keys_max, merge);
  const int kpw = plan.kpw, chunk_keys = 4 * kpw, nch = plan.nch, ll = plan.ll;
  if (relay) {
    if (!epoch || !status || spin_limit < 0 || (qw && !qk_ssq)) return O355_EINVAL;
    if (!plan.merge_in_kernel || H * hd > 8192 || Hkv * hd > 8192 || ((H * hd) & 127) || ((Hkv * hd) & 127)) return O355_EUNSUPPORTED;
  }
#define FUSED(HDv, QVv)                                                                                                 \
  if (kpw == 64) { FUSED_KPW(HDv, QVv, 64, false); } else if (kpw == 48) { FUSED_KPW(HDv, QVv, 48, false); } else { FUSED_KPW(HDv, QVv, 32, false); } \
  if (!tickets)                                                                                                        \
  hipLaunchKernelGGL((attn_decode_combine_kernel<O355_BF16, HDv>), dim3(H, B), dim3(HDv), 0, s, (const float*)ws, out, \
                     H, past_len, past_len_dev, nch, chunk_keys)
#define FUSED_RELAY(HDv)                                                                                                \
  if (kpw == 64) { FUSED_KPW(HDv, 1, 64, true); } else if (kpw == 48) { FUSED_KPW(HDv, 1, 48, true); } else { FUSED_KPW(HDv, 1, 32, true); }
#define FUSED_KPW(HDv, QVv, KPWv, RELAYv)                                                                               \
  hipLaunchKernelGGL((attn_decode_fused_kernel<HDv, QVv, KPWv, RELAYv>), dim3(nch, H, B), dim3(256), 0, s, (const uint16_t*)qkv,   \
                     (const uint16_t*)qw, (const uint16_t*)kw, sin_tab, cos_tab, (uint16_t*)kcache, (uint16_t*)vcache, \
                     key_bias, (float*)ws, H, Hkv, Lmax, n_pos, past_len, past_len_dev, nch, bias_stride, eps,         \
                     (const float*)qk_ssq, rope_now, (uint16_t*)out, tickets, ll, epoch, status, spin_limit, hint_in, hint_out)
  // the workspace starts with one ticket counter per (batch, head): zero on entry (zeroed at allocation,
  // reset by the workgroup that draws the last ticket), then one launch counter per (batch, head) for the flag
  // form (a region of its own: a workspace may serve both forms in turn), then the partials
  int* tickets = plan.merge_in_kernel ? reinterpret_cast<int*>(ws) : nullptr;
  ws = reinterpret_cast<float*>(ws) + (int64_t)2 * B * H;
  const int qv = (H * hd / 8 + 255) / 256;
  if (relay) {
    if (hd == 128) { FUSED_RELAY(128) } else { FUSED_RELAY(64) }
  } else if (hd == 128) {
    if (qv <= 1) { FUSED(128, 1); } else if (qv <= 2) { FUSED(128, 2); } else { FUSED(128, 4); }
  } else {
    if (qv <= 1) { FUSED(64, 1); } else if (qv <= 2) { FUSED(64, 2); } else { FUSED(64, 4); }
  }
#undef FUSED
#undef FUSED_RELAY
#undef FUSED_KPW
  O355_CHECK_LAUNCH();
}
}  // namespace

extern "C" int olmo355_attn_decode_fused_merge(const void* qkv, const void* qw, const void* kw, const float* sin_tab,
                                               const float* cos_tab, void* kcache, void* vcache, const float* key_bias,
                                               void* out, void* ws, int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax, int n_pos,
                                               int past_len, const int32_t* past_len_dev, int n_keys_max,
                                               int bias_stride, float eps, const float* qk_ssq, const float* rope_now,
                                               int dtype, int merge, void* stream) {
  return attn_fused_any(qkv, qw, kw, sin_tab, cos_tab, kcache, vcache, key_bias, out, ws, ws_bytes, B, H, Hkv, hd, Lmax, n_pos, past_len,
                        past_len_dev, n_keys_max, bias_stride, eps, qk_ssq, rope_now, dtype, merge, false, nullptr, nullptr, 0, nullptr, nullptr, stream);
}

extern "C" int olmo355_attn_decode_fused(const void* qkv, const void* qw, const void* kw, const float* sin_tab,
                                         const float* cos_tab, void* kcache, void* vcache, const float* key_bias,
                                         void* out, void* ws, int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax, int n_pos,
                                         int past_len, const int32_t* past_len_dev, int n_keys_max, int bias_stride,
                                         float eps, const float* qk_ssq, const float* rope_now, int dtype,
                                         void* stream) {
  return olmo355_attn_decode_fused_merge(qkv, qw, kw, sin_tab, cos_tab, kcache, vcache, key_bias, out, ws, ws_bytes, B, H, Hkv, hd,
                                         Lmax, n_pos, past_len, past_len_dev, n_keys_max, bias_stride, eps, qk_ssq,
                                         rope_now, dtype, -1, stream);
}

extern "C" int olmo355_attn_decode_relay(const uint32_t* qkv, const void* qw, const void* kw, const float* sin_tab,
                                         const float* cos_tab, void* kcache, void* vcache, const float* key_bias,
                                         uint32_t* out, void* ws, int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax, int n_pos,
                                         int past_len, const int32_t* past_len_dev, int n_keys_max, int bias_stride,
                                         float eps, const uint32_t* qk_ssq, const float* rope_now, const int32_t* epoch,
                                         int32_t* status, const int32_t* hint_in, int32_t* hint_out, int spin_limit,
                                         void* stream) {
  return attn_fused_any(qkv, qw, kw, sin_tab, cos_tab, kcache, vcache, key_bias, out, ws, ws_bytes, B, H, Hkv, hd, Lmax, n_pos, past_len,
                        past_len_dev, n_keys_max, bias_stride, eps, qk_ssq, rope_now, O355_BF16, -1, true, epoch, status,
                        spin_limit, hint_in, hint_out, stream);
}

// What a launch of olmo355_attn_decode_relay takes of the chip (as olmo355_w4_relay_footprint): out[0] workgroups,
// out[1] waves per workgroup, out[2] vector registers per lane, out[3] bytes of LDS per workgroup.
extern "C" int olmo355_attn_decode_relay_footprint(int B, int H, int hd, int n_keys_max, int* out) {
  if (!out || B <= 0 || H <= 0 || n_keys_max <= 0) return O355_EINVAL;
  if (hd != 128 && hd != 64) return O355_EUNSUPPORTED;
  const FusedPlan plan = fused_plan(B, H, n_keys_max, -1);
  if (!plan.merge_in_kernel) return O355_EUNSUPPORTED;
  out[0] = plan.nch * H * B, out[1] = 4;
  const void* fn = nullptr;
#define FP(HDv, KPWv) fn = reinterpret_cast<const void*>(attn_decode_fused_kernel<HDv, 1, KPWv, true>)
  if (hd == 128) {
    if (plan.kpw == 64) FP(128, 64); else if (plan.kpw == 48) FP(128, 48); else FP(128, 32);
  } else {
    if (plan.kpw == 64) FP(64, 64); else if (plan.kpw == 48) FP(64, 48); else FP(64, 32);
  }
#undef FP
  hipFuncAttributes fa;
  if (hipFuncGetAttributes(&fa, fn) != hipSuccess) return O355_ELAUNCH;
  out[2] = fa.numRegs, out[3] = (int)fa.sharedSizeBytes;
  return O355_OK;
}
