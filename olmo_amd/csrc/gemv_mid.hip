// int4 linear for up to 64 activation rows (the dispatcher sends it every product above 16 rows and the wide
// ones from 5): y[M,N] = x[M,K] . W[K,N], bf16 in and out.
//
// At these sizes the weight stream (N*K/2 bytes from HBM) and the activations (M*K*2 bytes, which
// every workgroup needs in full) are of the same order, and the vector ALU (unpacking nibbles,
// applying scales) is as scarce as memory.  A workgroup owns 2*NP column tiles of 16 and walks K in
// stages of GS groups of 128.  The stage's activations go from memory (L2) straight into LDS
// (buffer loads with the LDS destination, no registers, no ALU work), one stage ahead of their
// use.  A wave owns one pair of column tiles and one group of the stage, for all rows, so a weight
// word is unpacked once per workgroup; its weight pieces go from memory to registers two stages
// ahead.  Per group the matrix cores give T[n][m] = sum_k (128+q[k][n]) * x[m][k]
// (v_mfma_f32_16x16x32_bf16, weights as the A operand, 0x4300|q == 128+q exactly) and
// X[m] = sum_k x[m][k] (A = all ones), and the fp32 update
// acc += scale[n] * (T - (128 + zero[n]) * X[m]) applies scale and zero in fp32.  The GS waves
// that share columns are summed through LDS in fixed order: no atomics, nothing depends on
// scheduling.
#include <type_traits>

#include "common.h"

namespace {

template <int MT, int NP, int GS>
struct MidCfg {
  static constexpr int WAVES = NP * GS, NTHR = WAVES * 64;
  static constexpr int STAGE_K = GS * 128;
  static constexpr int KSEGS = 2 * GS;                   // 64-column segments per stage
  static constexpr int XBYTES = MT * 16 * STAGE_K * 2;   // one stage of activations
  static constexpr int XPW = XBYTES / 1024 / WAVES;      // 1 KiB copy instructions per wave per stage
  static constexpr int RED_BYTES = WAVES * 2 * MT * 1024;
  static constexpr int LDS_BYTES = 2 * XBYTES > RED_BYTES ? 2 * XBYTES : RED_BYTES;
  static constexpr int D = 2;                            // weight prefetch depth in stages
  static constexpr int KEEP = 6;                         // loads of one weight prefetch (2 tiles x piece, scales, zeros)
  static_assert((XBYTES / 1024) % WAVES == 0 && XPW % 2 == 0, "copy instructions per wave");
};

// LDS layout of a stage: blocks of 16 rows x 64 columns (2 KiB) indexed [row tile][segment]; a row is
// 128 bytes = 8 chunks of 16, and chunk c of row r sits at position c ^ ((r >> 1) & 7).  A copy
// instruction moves half a block (8 rows): 8 neighbouring lanes read one 128-byte line of x, and
// the 16 lanes (rows) of an operand read hit 16 different bank groups.
template <int MT, int NP, int GS>
__global__ __launch_bounds__(NP* GS * 64) void w4_mid_kernel(const uint16_t* __restrict__ x,
                                                            const uint32_t* __restrict__ wt,
                                                            const uint16_t* __restrict__ st,
                                                            const uint8_t* __restrict__ zt,
                                                            uint16_t* __restrict__ y, int M, int N, int K) {
  using C = MidCfg<MT, NP, GS>;
  constexpr int D = C::D;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int gi = wave % GS, pi = wave / GS;
  const int G = K >> 7, ntiles = N >> 4;
  const int NS = (G + GS - 1) / GS;
  const int tile0 = ((int)blockIdx.x * NP + pi) * 2;
  const int m16 = lane & 15, kq = lane >> 4;
  const UnpackConsts uc;
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

  // ---- activations: memory -> LDS, one stage ahead.  Copy instruction q = wave*XPW + j covers half
  // h = q & 1 of block q >> 1; rows past M and columns past K arrive as zeros (buffer bounds).
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(x, (int64_t)M * K * 2);
  uint32_t x_lane[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r16 = 8 * h + (lane >> 3);
    x_lane[h] = (uint32_t)(r16 * K + (((lane & 7) ^ ((r16 >> 1) & 7)) << 3)) * 2u;
  }
  auto copy_x = [&](int s, int buf) {
#pragma unroll
    for (int j = 0; j < C::XPW; ++j) {
      const int q = wave * C::XPW + j, blk = q >> 1;
      const int rt = blk / C::KSEGS, kseg = blk % C::KSEGS;
      const int k0 = s * C::STAGE_K + kseg * 64;
      const uint32_t voff = k0 < K ? x_lane[j & 1] + (uint32_t)(rt * 16 * K) * 2u : 0x80000000u;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)(smem + buf * C::XBYTES + q * 1024), 16, voff, k0 * 2, 0, 0);
    }
  };
  // operand reads: lane (m16, kq), k-step t of group gi -> segment 2*gi + t/2, chunk 4*(t&1) + kq
  int x_rd[2];
#pragma unroll
  for (int o = 0; o < 2; ++o) x_rd[o] = gi * 4096 + m16 * 128 + (((4 * o + kq) ^ ((m16 >> 1) & 7)) << 4);

  // ---- weights: D stages in flight per wave; groups past K load nothing (zeros)
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(wt, (int64_t)ntiles * G * 1024), rs = make_rsrc(st, (int64_t)ntiles * G * 32),
                               rz = make_rsrc(zt, (int64_t)ntiles * G * 8);
  u32x4 w[D][2];
  u32x2 sv[D][2];
  uint32_t zv[D][2];
  int tbase[2];
#pragma unroll
  for (int e = 0; e < 2; ++e) tbase[e] = min(tile0 + e, ntiles - 1) * G;  // out-of-range tiles: computed, dropped
  auto issue_w = [&](int slot, int s) {
    const int g = s * GS + gi;
    const uint32_t dead = g < G ? 0u : 0x80000000u;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int t = tbase[e] + g;
      w[slot][e] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, dead + lane * 16, t * 1024, 0));
      sv[slot][e] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rs, dead + kq * 8, t * 32, 0));
      zv[slot][e] = __builtin_amdgcn_raw_buffer_load_b16(rz, dead + kq * 2, t * 8, 0);
    }
  };

  f32x4 acc[2][MT];
#pragma unroll
  for (int e = 0; e < 2; ++e)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[e][mt] = zero4;

  const bf16x8 ones = __builtin_bit_cast(bf16x8, u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u});
  auto compute = [&](int slot, int buf) {
    f32x4 tmp[2][MT], xsum[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      xsum[mt] = zero4;
#pragma unroll
      for (int e = 0; e < 2; ++e) tmp[e][mt] = zero4;
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      bf16x8 xb[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        xb[mt] = *reinterpret_cast<const bf16x8*>(smem + buf * C::XBYTES + x_rd[t & 1] + (mt * C::KSEGS + (t >> 1)) * 2048);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xsum[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, xb[mt], xsum[mt], 0, 0, 0);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const bf16x8 a = unpack_w4_bias128(w[slot][e][t], uc);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) tmp[e][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, xb[mt], tmp[e][mt], 0, 0, 0);
      }
    }
#pragma unroll
    for (int e = 0; e < 2; ++e)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t sp = sv[slot][e][i >> 1];
        const uint16_t sb = (uint16_t)((i & 1) ? (sp >> 16) : (sp & 0xffffu));
        const float sc = (float)__builtin_bit_cast(_Float16, sb);
        const float nzc = -(float)(129 + (int)((zv[slot][e] >> (4 * i)) & 15u));  // -(128 + (stored + 1))
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[e][mt][i] = __builtin_fmaf(sc, __builtin_fmaf(nzc, xsum[mt][0], tmp[e][mt][i]), acc[e][mt][i]);
      }
  };

  // Every stage issues the same loads in the same order (past the end they are out of bounds and
  // move nothing), so "at most KEEP loads outstanding" always means: this stage's activations have
  // landed, the weight prefetch issued after them may still be in flight.
  auto stage = [&](int s, auto slot_c) {
    constexpr int slot = decltype(slot_c)::value;
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(C::KEEP, true));
    lds_barrier();  // stage s is in LDS for everyone; everyone is done reading the other buffer
    copy_x(s + 1, (s + 1) & 1);
    compute(slot, s & 1);
    issue_w(slot, s + D);
  };

  // issue order: the first weight prefetch, the first activations, then one prefetch per stage
  issue_w(0, 0);
  copy_x(0, 0);
  issue_w(1, 1);
  int s = 0;
  for (; s + 1 < NS; s += 2) {
    stage(s, std::integral_constant<int, 0>{});
    stage(s + 1, std::integral_constant<int, 1>{});
  }
  if (s < NS) stage(s, std::integral_constant<int, 0>{});

  // ---- sum the GS waves that share columns, in fixed order
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, true));  // the copies past the end still write (zeros) into LDS
  lds_barrier();
  float* red = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int e = 0; e < 2; ++e)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave * (2 * MT * 256) + ((e * MT + mt) * 4 + i) * 64 + lane] = acc[e][mt][i];
  lds_barrier();
  for (int cmb = gi; cmb < 2 * MT; cmb += GS) {
    const int e = cmb / MT, mt = cmb % MT;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g2 = 0; g2 < GS; ++g2) {
      const int w2 = g2 + GS * pi;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] += red[w2 * (2 * MT * 256) + (cmb * 4 + i) * 64 + lane];
    }
    const int m = mt * 16 + m16;
    if (m < M && tile0 + e < ntiles) {
      u32x2 o;
      o.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
      o.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
      *reinterpret_cast<u32x2*>(y + (int64_t)m * N + (tile0 + e) * 16 + 4 * kq) = o;
    }
  }
}

template <int MT, int NP, int GS>
int launch_mid(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y, int M, int N,
               int K, hipStream_t stream) {
  using C = MidCfg<MT, NP, GS>;
  auto kern = w4_mid_kernel<MT, NP, GS>;
  if (C::LDS_BYTES > 48 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES) != hipSuccess)
    return O355_ELAUNCH;
  const int ntiles = N >> 4;
  const unsigned blocks = (unsigned)((ntiles + 2 * NP - 1) / (2 * NP));
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(C::NTHR), C::LDS_BYTES, stream, x, wt, st, zt, y, M, N, K);
  O355_CHECK_LAUNCH();
}

}  // namespace

// 1..64 rows; the caller has checked pointers and that K is a multiple of 128 and N of 16.
// pairs: column-tile pairs per workgroup, 0 = choose, 1 or 2.
int o355_w4_mid_dispatch(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                         int M, int N, int K, int pairs, void* stream) {
  if (M < 1 || M > 64 || (int64_t)M * K * 2 >= (1ll << 31) || (int64_t)(N >> 4) * (K >> 7) * 1024 >= (1ll << 31))
    return O355_EUNSUPPORTED;  // 32-bit buffer offsets
  hipStream_t s = as_stream(stream);
  const int quads = ((N >> 4) + 3) / 4;  // workgroups with four column tiles each
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  int np = quads >= (mt == 1 ? 512 : 128) ? 2 : 1;
  if (pairs == 1 || pairs == 2) np = pairs;
  if (mt == 1) return np == 2 ? launch_mid<1, 2, 4>(x, wt, st, zt, y, M, N, K, s) : launch_mid<1, 1, 4>(x, wt, st, zt, y, M, N, K, s);
  if (mt == 2) return np == 2 ? launch_mid<2, 2, 4>(x, wt, st, zt, y, M, N, K, s) : launch_mid<2, 1, 4>(x, wt, st, zt, y, M, N, K, s);
  return np == 2 ? launch_mid<4, 2, 4>(x, wt, st, zt, y, M, N, K, s) : launch_mid<4, 1, 4>(x, wt, st, zt, y, M, N, K, s);
}
