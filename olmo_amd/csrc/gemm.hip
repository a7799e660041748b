// Large-M linear layers (prefill): y[M,N] = x[M,K] . W[K,N] on the matrix cores
// (v_mfma_f32_16x16x32_bf16: with random operands it sustains 2.09 PFLOP/s on this part where
// v_mfma_f32_32x32x16_bf16 sustains 1.85 -- the chip is power-bound and the smaller tile moves fewer
// accumulator registers per flop), fp32 accumulation, bf16 output.
//
// Workgroup = 8 waves (two per SIMD) in a 2x4 or 4x2 arrangement over a BM x BN output tile: 256 rows by
// 256, 192 or 128 columns, or 128 rows by 128 or 64 columns; each wave owns 2 WMT x 2 WNT MFMA tiles of
// 16 x 16.  K advances 64 per stage, two k-steps of 32.  Activations go memory -> LDS directly (8 rows x 128
// bytes per instruction, the 16-byte chunks of a row XOR-swizzled so the operand reads are conflict-free), ring of
// three stages requested two stages ahead.  Weights are staged in LDS in *fragment-major* order
// -- [16-column tile][k-step of 32][64 lanes][16 bytes], which is the order of the tiled weight formats themselves --
// so every MFMA operand is one conflict-free ds_read_b128; int4 words come into registers two stages ahead and are
// dequantised (scale and zero in fp32, one rounding to bf16) into LDS ahead of their stage, double-buffered; dense
// weights are copied memory -> LDS as they are tiled.  The staging work is spread between the k-steps of the
// MFMA loop so that the VALU / LDS / memory instructions issue in the shadow of the matrix pipeline; operand
// fragments are read ahead of the matrix instructions that use them into registers that have just been read for
// the last time; one barrier per stage, where the stage's last fragments have been asked for.  The matrix
// instructions take the weight fragment as their first operand, so the accumulators hold the output tile transposed
// (a lane owns four neighbouring columns of one row per 16 x 16 block) and the epilogue, after one exchange of
// half-rows between neighbouring blocks, writes 16 bytes per lane and store.
//
// The int4 operand is W = bf16(scale * (q - zero)) (fp32 product, one rounding).
#include "common.h"
#include <algorithm>
#include <type_traits>

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int BK = 64;      // K per stage
constexpr int KSTEPS = 2;   // MFMA k-steps of 32 per stage

// dequantise one tiled word (8 weights of one column) to 8 bf16 in MFMA operand order.
// The nibbles are turned into fp16 numbers where they stand: (w & 0x000f000f) | 0x64006400 is the pair
// (1024 + q_lo, 1024 + q_hi), and the same with the mask one nibble up the pair (1024 + 16 q); a mixed-precision
// fma takes either half as it is.  s * (1024 + q) + c0 with c0 = -(1024 + zero) * s, and (s / 16) * (1024 + 16 q)
// + c1 with c1 = -(64 + zero) * s: every product and sum is exact in fp32 (11 x 11 bits), so the value is
// s * (q - zero) with the single rounding to bf16 at the end.
struct DequantConsts { float s, c0, s16, c1; };
__device__ __forceinline__ DequantConsts dequant_consts(float s, int zero) {
  return {s, -(float)(1024 + zero) * s, s * 0.0625f, -(float)(64 + zero) * s};
}
__device__ __forceinline__ u32x4 dequant_word_bf16(uint32_t w, const DequantConsts& d) {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  auto pair = [](uint32_t p, float sm, float cm) {
    const f16x2 h = __builtin_bit_cast(f16x2, p);
    return pack_bf16x2(__builtin_fmaf((float)h[0], sm, cm), __builtin_fmaf((float)h[1], sm, cm));
  };
  // (w & mask) | magic in one instruction: it takes one scalar operand only, so the magic sits in a vector register
  auto and_or = [](uint32_t v, uint32_t mask, uint32_t magic) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "s"(mask), "v"(magic));
    return r;
  };
  const uint32_t w8 = w >> 8, magic = 0x64006400u;
  u32x4 o;
  o[0] = pair(and_or(w, 0x000f000fu, magic), d.s, d.c0);
  o[1] = pair(and_or(w, 0x00f000f0u, magic), d.s16, d.c1);
  o[2] = pair(and_or(w8, 0x000f000fu, magic), d.s, d.c0);
  o[3] = pair(and_or(w8, 0x00f000f0u, magic), d.s16, d.c1);
  return o;
}

template <bool F16>
__device__ __forceinline__ f32x4 mma16(const bf16x8& a, const bf16x8& b, const f32x4& c) {
  if constexpr (F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
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

// SWIGLU (int4, WNT == 2): the weight holds [up | gate] column halves of N/2 each; a tile's first 32-column
// block per wave comes from the up half and its second from the matching gate columns, so both land in
// the same lanes and the epilogue writes silu(gate) * up, [M, N/2] (SwiGLU.forward, olmo/model.py:365-368).
//
// SPLIT: the launch has gridDim.y workgroups per tile, each over its own run of K (whole units of 256, dealt
// evenly), writing fp32 partial tiles to part[split][M][N]; splitk_reduce_kernel adds them in split order and
// rounds once.  For launches with fewer tiles than CUs: the K loop is a serial chain of stages of about half a
// microsecond each, so a tile count of 64 leaves three quarters of the chip idle for K / 64 such stages.
// STREAMK: a workgroup of a grid that stays (one per CU) is handed segments -- a tile and a run of K -- one after
// the other.  sk_mode says what becomes of the accumulators: 0: the run is the tile's whole K, write the output;
// 1: leave the fp32 partial in this workgroup's slot and raise its flag; 2: add the partials of workgroups
// sk_first .. sk_self - 1, then write the output.  What the hand-over needs beyond that is read from the kernel's
// argument block when it is needed (StreamKArgs is the kernel's only parameter), so that none of it occupies
// registers during the K loop.
struct StreamKArgs {
  const uint16_t* x;
  const uint32_t* wt;
  const uint16_t* st;
  const uint8_t* zt;
  uint16_t* y;
  float* slots;    // [grid][8 waves][128 registers / 4][64 lanes] float4: a wave's accumulators as they stand
  int* flags;      // [grid]: the epoch of the launch whose partial the slot holds; word 513: status
  int M, N, K, tiles_n, tiles;
  int spin_limit;  // polls of a flag before a finishing workgroup gives up and writes NaN
  int publish;     // 0 (tests of the give-up path only): leave the flag down
  int epoch;       // this launch's flag value: differs from that of the launch before on the same workspace, never 0
};
typedef const __attribute__((address_space(4))) StreamKArgs* StreamKArgsPtr;
__device__ __forceinline__ StreamKArgsPtr streamk_args() {
  StreamKArgsPtr p = (StreamKArgsPtr)__builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(p));  // read again wherever it is used
  return p;
}
enum { GEMM_PLAIN = 0, GEMM_SPLIT = 1, GEMM_STREAMK = 2 };
constexpr int kStreamKStatusWord = O355_STREAMK_STATUS_WORD;  // int32 index in the workspace: epoch of a launch that gave up

// F16: the activations, the weights (dense, or int4 dequantised) and the output are fp16 instead of bf16 (plain tiles only)
template <int WAVES_M, int WAVES_N, int WMT, int WNT, bool W4, bool SWIGLU = false, int KIND = GEMM_PLAIN, bool F16 = false>  // wave grid, 32 x 32 blocks (of four 16 x 16 MFMA tiles) per wave
__device__ __forceinline__ void gemm_body(const uint16_t* __restrict__ x, const uint32_t* __restrict__ wt,
                                          const uint16_t* __restrict__ st, const uint8_t* __restrict__ zt,
                                          uint16_t* __restrict__ y, int M, int N, int K, int tile_m, int tile_n,
                                          int k0, int Kn,  // this workgroup's run of K (whole units of 256 unless all of K)
                                          float* __restrict__ part = nullptr, int sk_mode = 0, int sk_self = 0,
                                          int sk_first = 0, bool sk_raise = false, bool sk_defer = false) {
  constexpr bool SPLIT = KIND == GEMM_SPLIT;
  static_assert(!F16 || (!SWIGLU && KIND == GEMM_PLAIN), "fp16 activations: the plain tiles only");
  constexpr int NW = WAVES_M * WAVES_N, NT = 64 * NW;
  constexpr int BM = 32 * WMT * WAVES_M, BN = 32 * WNT * WAVES_N;
  constexpr int MT = 2 * WMT, NT16 = 2 * WNT;  // 16 x 16 MFMA tiles per wave
  constexpr int A_BLK = BM / 8;        // 1 KiB blocks per stage: activations, 8 rows x 128 bytes each
  constexpr int B_BLK = BN / 8;        // weights: 32x16 bf16 pieces (either layout)
  constexpr int A_PW = A_BLK / NW, B_PW = B_BLK / NW;
  // int4: (16-column tile, lane) items per thread per group of 128 rows; when the tiles do not divide
  // evenly among the waves the last item exists on the first waves only
  constexpr int B_ITEMS = (BN / 16 + NW - 1) / NW;
  constexpr bool B_RAGGED = (BN / 16) % NW != 0;
  static_assert(A_BLK % NW == 0 && B_BLK % NW == 0, "tile / wave split");
  extern __shared__ __align__(16) unsigned char smem[];
  u32x4* lds_a = reinterpret_cast<u32x4*>(smem);  // [3][A_BLK][64]: ring of three stages
  u32x4* lds_b = lds_a + 3 * A_BLK * 64;          // [2][B_BLK][64]

  int tid_ = threadIdx.x;
  // stream-K calls this once per segment inside a loop: what depends on the thread id only must be worked out again
  // per segment, or it is all kept in registers across the K loops (and accumulators are spilled to make room)
  if constexpr (KIND == GEMM_STREAMK) asm volatile("" : "+v"(tid_));
  const int tid = tid_, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  static_assert(!SWIGLU || (W4 && WNT == 2), "fused SwiGLU: int4 weights, two column blocks per wave");
  const int m0 = tile_m * BM, nt0 = SWIGLU ? 0 : tile_n * (BN / 16);  // fused: absolute tile indices, see tile_abs
  const int ntiles = N >> 4;
  // 16-column tile of the weight behind local tile ntl (32-column block ntl/2 = wave column wn = ntl/4, block j)
  auto tile_abs = [&](int ntl) {
    if constexpr (!SWIGLU) return ntl;
    const int ct = ntl >> 1, j = ct & 1, wn_ = ct >> 1;
    return (j ? (ntiles >> 1) : 0) + tile_n * (BN / 32) + wn_ * 2 + (ntl & 1);
  };
  const int G = K >> 7, KS = K >> 5;  // strides of the tiled weight: always of the whole K
  const int Gn = Kn >> 7;             // groups of 128 rows in the run
  const int stages = Kn / BK;
  const int row16 = lane & 15, kq4 = lane >> 4;  // operand row (or column) of a 16 x 32 fragment, its 8-wide k block

  // ---- activations: memory -> LDS directly ------------------------------------------------------
  // One instruction moves 8 rows x 128 bytes (the 64 k of a stage): 8 consecutive lanes cover one
  // row's cache line.  LDS keeps the rows 128 bytes apart with the 16-byte chunks of row r stored at
  // position chunk ^ ((r >> 1) & 7), which makes the MFMA operand reads (32 rows, one chunk) hit
  // every bank once; the swizzle is applied on the memory side because the LDS side of these loads
  // is lane-linear.
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(x + (int64_t)m0 * K + k0, ((int64_t)(M - m0) * K - k0) * 2);
  int a_voff[A_PW];
#pragma unroll
  for (int i = 0; i < A_PW; ++i) {
    const int row = 8 * (wave * A_PW + i) + (lane >> 3);
    const int c = (lane & 7) ^ ((row >> 1) & 7);
    a_voff[i] = (row * K + 8 * c) * 2;
  }
  auto load_a = [&](int s, int buf, int part = -1) {  // part: only the requests of that k-step's share
#pragma unroll
    for (int i = 0; i < A_PW; ++i)
      if (part < 0 || i * KSTEPS / A_PW == part)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)(smem + ((buf * A_BLK + wave * A_PW + i) << 10)), 16, a_voff[i],
                                               s * (BK * 2), 0, 0);
  };
  // operand read: lane (row16, kq4), 16-row tile rt, k-step ks -> 16-byte slot
  const int a_swz = (row16 >> 1) & 7;
  int a_rd[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) a_rd[ks] = row16 * 8 + ((4 * ks + kq4) ^ a_swz);

  // ---- weights ---------------------------------------------------------------------------------
  const int g0 = k0 >> 7, ks0 = k0 >> 5;  // first group / 32-row step of the run
  const __amdgpu_buffer_rsrc_t rw =
      W4 ? make_rsrc(wt + ((int64_t)nt0 * G + g0) * 256, ((int64_t)(ntiles - nt0) * G - g0) * 1024)
         : make_rsrc(wt + ((int64_t)nt0 * KS + ks0) * 256, ((int64_t)(ntiles - nt0) * KS - ks0) * 1024);
  const __amdgpu_buffer_rsrc_t rs_ = make_rsrc(W4 ? st + ((int64_t)nt0 * G + g0) * 16 : x, W4 ? ((int64_t)(ntiles - nt0) * G - g0) * 32 : 0);
  const __amdgpu_buffer_rsrc_t rz_ = make_rsrc(W4 ? zt + ((int64_t)nt0 * G + g0) * 8 : (const uint8_t*)x, W4 ? ((int64_t)(ntiles - nt0) * G - g0) * 8 : 0);
  // int4: one 16-byte piece (4 tiled words = the lane's share of a 128-row group), scale and zero per
  // item, fetched a group ahead into registers and dequantised on the way into LDS, fragment-major:
  // piece of lane l (column l&15 of its 16-column tile, rows 8*(l>>4).. of 32-row step j) goes to
  // fragment (tile/2, k-step 2j + (l>>5)), slot ((l>>4)&1)*32 + (tile&1)*16 + (l&15).
  constexpr int NBI = W4 ? B_ITEMS : 1;
  u32x4 rbw[2][NBI];
  uint32_t rsb[2][NBI], rzb[2][NBI];
  int bw_voff[NBI], bs_voff[NBI], bz_voff[NBI];
  if constexpr (W4) {
#pragma unroll
    for (int i = 0; i < B_ITEMS; ++i) {
      const int nta = tile_abs(wave + NW * i), col = lane & 15;
      bw_voff[i] = (nta * G * 64 + lane) * 16;
      bs_voff[i] = (nta * G * 16 + col) * 2;
      bz_voff[i] = nta * G * 8 + (col >> 1);
    }
  }
  auto fetch_b = [&](int g, int set, int part = -1) {  // part: as for the activations
#pragma unroll
    for (int i = 0; i < NBI; ++i) {
      if (part >= 0 && (2 * i + 1) * KSTEPS / (2 * NBI) != part) continue;
      rbw[set][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, bw_voff[i], g * 1024, 0));
      // kept raw: converting here would make the wave wait for the loads it has just issued
      rsb[set][i] = __builtin_amdgcn_raw_buffer_load_b16(rs_, bs_voff[i], g * 32, 0);
      rzb[set][i] = __builtin_amdgcn_raw_buffer_load_b8(rz_, bz_voff[i], g * 8, 0);
    }
  };
  auto stash_b_word = [&](int buf, int set, int i, int j) {  // word j (32-row step j of the group) of item i
    const int ntl = wave + NW * i;
    if (B_RAGGED && ntl >= BN / 16) return;  // wave-uniform
    const int zero = 1 + (int)((rzb[set][i] >> (4 * (lane & 1))) & 15u);  // stored zero points are one less
    // a tiled word is already the lane's piece of a 16-column x 32-row operand fragment: it stays in its lane
    if constexpr (F16) {
      lds_b[(buf * B_BLK + ntl * KSTEPS + (j & 1)) * 64 + lane] = dequant_word_f16(rbw[set][i][j], dequant_consts_f16((uint16_t)rsb[set][i], zero));
    } else {
      const float sc = (float)__builtin_bit_cast(_Float16, (uint16_t)rsb[set][i]);
      lds_b[(buf * B_BLK + ntl * KSTEPS + (j & 1)) * 64 + lane] = dequant_word_bf16(rbw[set][i][j], dequant_consts(sc, zero));
    }
  };
  // dense: the tiled pieces [16-column tile][32-row step][64][16 B] are copied as they are
  int bd_voff[W4 ? 1 : B_PW];
  if constexpr (!W4) {
#pragma unroll
    for (int i = 0; i < B_PW; ++i) {
      const int q = wave * B_PW + i;
      bd_voff[i] = (((q >> 1) * KS + (q & 1)) * 64 + lane) * 16;
    }
  }
  auto load_b_dense = [&](int s, int buf) {
#pragma unroll
    for (int i = 0; i < (W4 ? 0 : B_PW); ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(smem + ((3 * A_BLK + buf * B_BLK + wave * B_PW + i) << 10)), 16,
                                               bd_voff[i], s * 2048, 0, 0);
  };
  // operand read of 16-column tile ct, k-step ks: either kind of weight sits in LDS as [tile][k-step][64 lanes][16 B]
  const int b_rd = lane;
  auto b_slot = [&](int ct, int ks) { return (ct * KSTEPS + ks) * 64; };

  // The stage's one barrier stands where its last operand fragments have been asked for: at the end of the k-step
  // before the last when a k-step's fragments all sit in registers at once (they are then asked for one k-step
  // ahead), otherwise inside the last k-step, after the RB rounds whose registers are refilled from this stage.
  constexpr int MT_ = 2 * WMT, NT16_ = 2 * WNT, OUT_ = NT16_ <= MT_ ? MT_ : NT16_;
  constexpr int RB = OUT_ > 4 ? OUT_ - 4 : 0;
  constexpr int LAST_PART = RB > 0 ? KSTEPS - 1 : KSTEPS - 2;  // requests of a stage issued up to this k-step precede its barrier
  constexpr int keep_a = [] { int n = 0; for (int i = 0; i < A_PW; ++i) n += (i * KSTEPS / A_PW <= LAST_PART); return n; }();
  constexpr int keep_b = [] { int n = 0; for (int i = 0; i < NBI; ++i) n += ((2 * i + 1) * KSTEPS / (2 * NBI) <= LAST_PART); return n; }();

  f32x4 acc[MT][NT16];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT16; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Operand fragments are read ahead of the matrix instructions that use them, into registers that have just
  // been read for the last time.  The k-step is a loop of rounds over the fragments of one operand (the one with
  // more of them), each round multiplying one of them with all fragments of the other.  The outer operand keeps at
  // most four fragments in registers: after round r its registers are asked for the fragment of round r + 4
  // (of this k-step or of the next); the inner operand's fragments are asked for again during the k-step's last
  // round.
  constexpr bool OUTER_A = NT16 <= MT;
  constexpr int OUT = OUTER_A ? MT : NT16, INN = OUTER_A ? NT16 : MT, OS = OUT < 4 ? OUT : 4;
  static_assert((KSTEPS * OUT) % OS == 0, "a stage's rounds must fill the slots a whole number of times");
  bf16x8 fo[OS], fi[INN];
  auto read_a = [&](int abuf, int i, int ks) {
    return __builtin_bit_cast(bf16x8, lds_a[abuf * A_BLK * 64 + (wm * MT + i) * 128 + a_rd[ks]]);
  };
  auto read_b = [&](int bbuf, int j, int ks) {
    return __builtin_bit_cast(bf16x8, lds_b[bbuf * B_BLK * 64 + b_slot(wn * NT16 + j, ks) + b_rd]);
  };
  auto read_outer = [&](int abuf, int bbuf, int t, int ks) { return OUTER_A ? read_a(abuf, t, ks) : read_b(bbuf, t, ks); };
  auto read_inner = [&](int abuf, int bbuf, int t, int ks) { return OUTER_A ? read_b(bbuf, t, ks) : read_a(abuf, t, ks); };
  auto ring_next = [](int ab) { return ab == 2 ? 0 : ab + 1; };
  // int4: a thread's 2 * B_ITEMS words of a stage are dequantised in the k-steps before the barrier that
  // publishes the stage, an equal share in each: see do_stage
  auto word_slot = [](int i) { return i * KSTEPS / (2 * B_ITEMS); };

  // One stage.  Activations sit in a ring of three LDS buffers and are requested two stages ahead;
  // the weights are double-buffered in LDS (int4: requested two stages ahead into registers, set
  // = parity of the 128-row group, and dequantised into LDS ahead of their stage; dense: copied one stage
  // ahead).  The stage's one barrier stands where the wave has asked for the stage's last fragments (inside the
  // last k-step when the outer operand has more fragments than register slots, else before it): from there on
  // the buffers of this stage may be written again, and everything of the next stage is in LDS, so the reads after
  // it fetch the next stage's first fragments.  A read of this stage placed after the barrier would race with the
  // faster waves' writes of the stage after next.  Memory operations complete in order, so waiting until only the
  // requests issued in this stage before the barrier's part (KEEP of them) are outstanding means that everything
  // the next stage reads has landed.
  //   h = parity of the stage = weight LDS buffer (and, int4, the half of the group)
  //   p = parity of the group (int4 register set)
  auto do_stage = [&](int s, int ab, auto hc, auto pc) {
    constexpr int h = decltype(hc)::value, p = decltype(pc)::value;
    const int s2 = min(s + 2, stages - 1);  // past the end: re-fetch the last stage into a buffer nobody reads
    const int ab1 = ring_next(ab), ab2 = ring_next(ab1);
    auto stage_barrier = [&]() {
      constexpr int KEEP = keep_a + ((W4 && h == 1) ? 3 * keep_b : 0);
      static_assert(KEEP < 64, "vmcnt range");
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt((KEEP & 15) | ((KEEP >> 4) << 14) | 0x0070);  // vmcnt(KEEP) lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    };
    if constexpr (!W4) {
      load_b_dense(min(s + 1, stages - 1), h ^ 1);
      __builtin_amdgcn_sched_barrier(0);  // keep the order: the weights' requests are the older ones
    }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const int nks = (ks + 1) & (KSTEPS - 1);
      const int nab = ks == KSTEPS - 1 ? ab1 : ab, nh = ks == KSTEPS - 1 ? (h ^ 1) : h;
      // requests are spread over the stage: a burst of them stalls the wave at issue
      load_a(s2, ab2, ks);
      if constexpr (W4 && h == 1) fetch_b(min((s >> 1) + 2, Gn - 1), p, ks);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = 0; r < OUT; ++r) {
        const int slot = (ks * OUT + r) % OS;  // rounds are numbered through the stage: slots rotate across its k-steps
#pragma unroll
        for (int q = 0; q < INN; ++q) {
          if constexpr (OUTER_A) acc[r][q] = mma16<F16>(fi[q], fo[slot], acc[r][q]);
          else acc[q][r] = mma16<F16>(fo[slot], fi[q], acc[q][r]);
          if (r == OUT - 1) fi[q] = read_inner(nab, nh, q, nks);
        }
        const int rn = r + OS;  // the round this slot serves next
        fo[slot] = rn < OUT ? read_outer(ab, h, rn, ks) : read_outer(nab, nh, rn - OUT, nks);
        if (RB > 0 && ks == KSTEPS - 1 && r == RB - 1) stage_barrier();  // the stage's last fragments have been asked for
      }
      if constexpr (W4) {
#pragma unroll
        for (int i = 0; i < 2 * B_ITEMS; ++i) {
          if (ks < KSTEPS - 1) {
            // next stage's words: second half of this group (h == 0) or first half of the next (h == 1)
            if (word_slot(i) == ks + 1) stash_b_word(h ^ 1, p ^ h, i >> 1, 2 * (h ^ 1) + (i & 1));
          } else {
            // after the barrier: first words of the stage after the next (same half, next group) into this stage's buffer
            if (word_slot(i) == 0) stash_b_word(h, p ^ 1, i >> 1, 2 * h + (i & 1));
          }
        }
      }
      if (RB == 0 && ks == KSTEPS - 2) stage_barrier();
    }
  };

  // ---- prologue: stages 0 and 1 of the activations, stage 0 of the weights -----------------------
  load_a(0, 0);
  load_a(min(1, stages - 1), 1);
  if constexpr (W4) {
    fetch_b(0, 0);
#pragma unroll
    for (int i = 0; i < 2 * B_ITEMS; ++i) stash_b_word(0, 0, i >> 1, i & 1);
#pragma unroll
    for (int i = 0; i < 2 * B_ITEMS; ++i)
      if (word_slot(i) == 0) stash_b_word(1, 0, i >> 1, 2 + (i & 1));  // what the k-step before stage 0 would have done
    fetch_b(min(1, Gn - 1), 1);
  } else {
    load_b_dense(0, 0);
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  if constexpr (KIND == GEMM_STREAMK) {
    // the partial this workgroup left in the segment before: every wave has just waited for all its memory
    // operations, those stores among them, so the flag can go up without a wait of its own
    if (sk_raise && tid == 0) {
      const StreamKArgsPtr ka = streamk_args();
      if (ka->publish) __hip_atomic_store(ka->flags + sk_self, ka->epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
#pragma unroll
  for (int t = 0; t < OS; ++t) fo[t] = read_outer(0, 0, t, 0);
#pragma unroll
  for (int t = 0; t < INN; ++t) fi[t] = read_inner(0, 0, t, 0);

  using H0 = std::integral_constant<int, 0>;
  using H1 = std::integral_constant<int, 1>;
  int s = 0, ab = 0;
  for (; s + 3 < stages; s += 4) {
    do_stage(s, ab, H0{}, H0{});
    ab = ring_next(ab);
    do_stage(s + 1, ab, H1{}, H0{});
    ab = ring_next(ab);
    do_stage(s + 2, ab, H0{}, H1{});
    ab = ring_next(ab);
    do_stage(s + 3, ab, H1{}, H1{});
    ab = ring_next(ab);
  }
  if (s < stages) {  // up to three stages left; s is a multiple of four, so the parities are known
    do_stage(s, ab, H0{}, H0{});
    ab = ring_next(ab);
    if (s + 1 < stages) {
      do_stage(s + 1, ab, H1{}, H0{});
      ab = ring_next(ab);
      if (s + 2 < stages) do_stage(s + 2, ab, H0{}, H1{});
    }
  }

  // ---- stream-K: partial tiles travel between workgroups as the accumulators stand ------------------------
  constexpr int QUADS = MT * NT16;  // float4 per lane: one per 16 x 16 block
  constexpr int SLOT_BYTES = NW * QUADS * 64 * 16;
  auto quad_off = [&](int i, int j) { return ((wave * QUADS + i * NT16 + j) * 64 + lane) * 16; };
  if constexpr (KIND == GEMM_STREAMK) {
    // (a partial is left behind -- sk_mode 1 -- from inside the ordinary epilogue's loops below: as a block of
    // its own before them it drives the register allocation of the whole function into spilling accumulators)
    if (sk_mode == 2) {
      const StreamKArgsPtr ka = streamk_args();
      float* const slots = ka->slots;
      int* const flags = ka->flags;
      const int spin_limit = ka->spin_limit, epoch = ka->epoch;
      // the workgroups first .. self - 1 hold the earlier runs of this tile's K and finished them before anything
      // else they had to do; their partials are added in a fixed order.  The wait is bounded: a flag that does
      // not show this launch's epoch within spin_limit polls turns the tile into NaN instead of hanging the grid,
      // and the status word of the workspace says so.  Flags are never cleared: the next launch waits for its
      // own epoch, so a flag raised late by a workgroup nobody waited for any more cannot be mistaken for news.
      int* s_ok = reinterpret_cast<int*>(smem);  // the operand buffers are done with once every wave is past the K loop
      for (int pc = sk_self - 1; pc >= sk_first; --pc) {
        __syncthreads();
        if (tid == 0) {
          int ok = 0;
          for (int spin = 0; spin <= spin_limit; ++spin) {
            if (__hip_atomic_load(flags + pc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == epoch) {
              ok = 1;
              break;
            }
            __builtin_amdgcn_s_sleep(8);
          }
          if (!ok) __hip_atomic_store(flags + kStreamKStatusWord, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          *s_ok = ok;
        }
        __syncthreads();
        const int ok = *s_ok;
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(reinterpret_cast<const char*>(slots) + (int64_t)pc * SLOT_BYTES, SLOT_BYTES);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          f32x4 v[NT16];
#pragma unroll
          for (int j = 0; j < NT16; ++j)
            v[j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, quad_off(i, j), 0, 16 /* sc1 */));
#pragma unroll
          for (int j = 0; j < NT16; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][e] = ok ? acc[i][j][e] + v[j][e] : __builtin_nanf("");
        }
      }
    }
  }

  // ---- epilogue ------------------------------------------------------------------------------------------
  // The products were formed as W^T-tile x X^T-tile, so a lane holds one output row m = lane & 15 of its 16 x 16
  // block and the four neighbouring columns n = 4 (lane >> 4) + r.  As bf16 pairs, two blocks that are neighbours along
  // n trade half-rows of the wave (v_permlane16_swap): the lanes of rows 0 and 2 end up with columns 0-7 and 8-15 of
  // the first block, those of rows 1 and 3 with the same of the second -- one 16-byte store per lane and pair of
  // blocks instead of eight 2-byte ones.
  // sk_mode 1: device-scope stores (they do not stay in this XCD's L2) of one block's accumulators into this
  // workgroup's slot; once all are out every wave waits for its own to be acknowledged, then one thread raises the flag
  auto leave_partial_block = [&](int i, int j) {
    const StreamKArgsPtr ka = streamk_args();
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(reinterpret_cast<const char*>(ka->slots) + (int64_t)sk_self * SLOT_BYTES, SLOT_BYTES);
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[i][j]), rs, quad_off(i, j), 0, 16 /* sc1 */);
  };
  auto announce_partial = [&]() {
    const StreamKArgsPtr ka = streamk_args();
    int* const flags = ka->flags;
    const int publish = ka->publish;
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));
    __syncthreads();
    if (tid == 0 && publish) __hip_atomic_store(flags + sk_self, ka->epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  // va, vb: this lane's four outputs (columns 4 kq4 .. + 3 of row m) of two blocks whose first columns are nb and nb + 16
  auto store_pair = [&](const f32x4& va, const f32x4& vb, uint16_t* __restrict__ dst, int m, int nb, int ncols, int ld) {
    uint32_t o[2][2];
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      const auto sw = F16 ? __builtin_amdgcn_permlane16_swap(pack_f16x2(va[2 * x], va[2 * x + 1]), pack_f16x2(vb[2 * x], vb[2 * x + 1]), false, false)
                          : __builtin_amdgcn_permlane16_swap(pack_bf16x2(va[2 * x], va[2 * x + 1]), pack_bf16x2(vb[2 * x], vb[2 * x + 1]), false, false);
      o[0][x] = sw[0], o[1][x] = sw[1];
    }
    const int n = nb + 16 * (kq4 & 1) + 8 * (kq4 >> 1);
    if (m < M && n < ncols) *reinterpret_cast<u32x4*>(dst + (int64_t)m * ld + n) = u32x4{o[0][0], o[0][1], o[1][0], o[1][1]};
  };
  if constexpr (SWIGLU) {
    // per wave: 16-column blocks 0, 1 come from the up half of the weight, 2, 3 from the matching gate columns
    const int half_n = N >> 1;
    const int nb = tile_n * (BN / 2) + wn * 32;  // no ragged columns: N/2 is a multiple of BN/2
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      if (KIND == GEMM_STREAMK && sk_mode == 1) {
#pragma unroll
        for (int j = 0; j < NT16; ++j) leave_partial_block(i, j);
        continue;
      }
      f32x4 v[2];
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float up = round_bf16(acc[i][jj][e]), gate = round_bf16(acc[i][jj + 2][e]);  // the Linear's bf16 output
          const float sg = round_bf16(gate / (1.f + expf(-gate)));
          v[jj][e] = sg * up;
        }
      store_pair(v[0], v[1], y, m0 + (wm * MT + i) * 16 + row16, nb, half_n, half_n);
    }
    if (KIND == GEMM_STREAMK && sk_mode == 1 && !sk_defer) announce_partial();
    return;
  }
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT16; j += 2) {
      if (KIND == GEMM_STREAMK && sk_mode == 1) {
        leave_partial_block(i, j);
        leave_partial_block(i, j + 1);
        continue;
      }
      const int nb = (nt0 >> 1) * 32 + (wn * NT16 + j) * 16;  // wave-uniform; columns come in whole blocks of 16
      if (nb >= N) continue;
      const int m = m0 + (wm * MT + i) * 16 + row16;
      if constexpr (SPLIT) {
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const int n = nb + 16 * jj + 4 * kq4;
          if (m < M && n < N) *reinterpret_cast<f32x4*>(part + ((int64_t)blockIdx.y * M + m) * N + n) = acc[i][j + jj];
        }
      } else {
        store_pair(acc[i][j], acc[i][j + 1], y, m, nb, N, N);
      }
    }
  if (KIND == GEMM_STREAMK && sk_mode == 1 && !sk_defer) announce_partial();
}

template <int WAVES_M, int WAVES_N, int WMT, int WNT, bool W4>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_splitk_kernel(const uint16_t* __restrict__ x,
                                                                            const uint32_t* __restrict__ wt,
                                                                            const uint16_t* __restrict__ st,
                                                                            const uint8_t* __restrict__ zt,
                                                                            float* __restrict__ part, int M, int N, int K,
                                                                            int tiles_m, int tiles_n) {
  int tile_m, tile_n;
  tile_of(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n);
  // this workgroup's run of K: whole units of 256, dealt evenly over gridDim.y
  const int units = K >> 8, z = blockIdx.y, nz = gridDim.y;
  const int u0 = units * z / nz, u1 = units * (z + 1) / nz;
  gemm_body<WAVES_M, WAVES_N, WMT, WNT, W4, false, GEMM_SPLIT>(x, wt, st, zt, nullptr, M, N, K, tile_m, tile_n, u0 << 8,
                                                              (u1 - u0) << 8, part);
}

// y = bf16(part[0] + part[1] + ... ) in that order, four outputs per thread
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const f32x4* __restrict__ part, u32x2* __restrict__ y,
                                                            int64_t n4, int splits) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  f32x4 a = part[i];
  for (int z = 1; z < splits; ++z) {
    const f32x4 b = part[z * n4 + i];
    a[0] += b[0], a[1] += b[1], a[2] += b[2], a[3] += b[3];
  }
  y[i] = u32x2{pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3])};
}

template <int WAVES_M, int WAVES_N, int WMT, int WNT, bool W4, bool SWIGLU = false, bool F16 = false>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_kernel(const uint16_t* __restrict__ x,
                                                                     const uint32_t* __restrict__ wt,
                                                                     const uint16_t* __restrict__ st,
                                                                     const uint8_t* __restrict__ zt,
                                                                     uint16_t* __restrict__ y, int M, int N, int K,
                                                                     int tiles_m, int tiles_n) {
  int tile_m, tile_n;
  tile_of(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n);
  gemm_body<WAVES_M, WAVES_N, WMT, WNT, W4, SWIGLU, GEMM_PLAIN, F16>(x, wt, st, zt, y, M, N, K, tile_m, tile_n, 0, K);
}

// Stream-K: a grid that stays, one workgroup per CU.  The tiles' K runs, in units of 256, form one sequence (tile
// after tile, consecutive tiles share their row panel); it is cut into gridDim.x equal pieces, so every CU does the
// same amount of matrix work whatever the tile count.  A piece is a run of segments: at most one tile whose K it
// only begins (or only continues: the piece lies inside one tile) -- done first, left as an fp32 partial in the
// workgroup's slot --, whole tiles, and at most one tile whose K it ends -- done last: it adds the partials of
// the workgroups before it, which were the first thing those did.  No workgroup waits for one that waits.
// Consecutive pieces go to the CUs of one XCD (workgroup ids go round-robin over the XCDs), so an XCD works on a
// band of consecutive tiles and their row panels stay in its L2.
template <int WAVES_M, int WAVES_N, int WMT, int WNT, bool W4, bool SWIGLU>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_streamk_kernel(StreamKArgs) {
  for (int i = 0;; ++i) {
    // everything about the piece is worked out again per segment from the argument block and the workgroup id
    // (a few scalar instructions) instead of being carried through the K loop
    const StreamKArgsPtr ka = streamk_args();
    const int tiles = ka->tiles, tiles_n = ka->tiles_n, K = ka->K;
    int bid = blockIdx.x;
    asm volatile("" : "+s"(bid));
    const int G = gridDim.x;
    const int c = (G & 7) == 0 ? (bid & 7) * (G >> 3) + (bid >> 3) : bid;
    const int KU = K >> 8;
    const int W = tiles * KU;  // the host keeps W * G below 2^31
    const int u0 = W * c / G, u1 = W * (c + 1) / G;
    if (u0 >= u1) break;
    const int t_first = u0 / KU, t_last = (u1 - 1) / KU;
    const bool tail_partial = (u1 % KU) != 0;                          // the last tile's K is only begun or continued
    const bool head_finish = (u0 % KU) != 0 && (t_first + 1) * KU <= u1;  // the first tile's K is ended here
    const int nseg = t_last - t_first + 1, nrest = nseg - (tail_partial ? 1 : 0);
    if (i >= nseg) break;
    int t;
    if (tail_partial && i == 0) {
      t = t_last;
    } else {
      const int j = i - (tail_partial ? 1 : 0);
      t = head_finish ? (j < nrest - 1 ? t_first + j + 1 : t_first) : t_first + j;
    }
    const int tb = t * KU;
    const int k_a = max(u0, tb) - tb, k_b = min(u1, tb + KU) - tb;
    const int mode = (k_a == 0 && k_b == KU) ? 0 : (k_b < KU ? 1 : 2);
    int first = c;
    if (mode == 2) {  // the workgroup whose piece holds the tile's first unit
      first = (int)((int64_t)tb * G / W);
      while (W * (first + 1) / G <= tb) ++first;
      while (W * first / G > tb) --first;
    }
    // A partial is always the first segment of a piece.  When more segments follow, its flag goes up after the next
    // segment's first barrier (which waits for all memory operations anyway) instead of after a wait of its own.
    const bool defer = mode == 1 && nseg > 1, raise = i == 1 && tail_partial;
    __syncthreads();  // every wave is done with the LDS buffers of the segment before
    gemm_body<WAVES_M, WAVES_N, WMT, WNT, W4, SWIGLU, GEMM_STREAMK>(ka->x, ka->wt, ka->st, ka->zt, ka->y, ka->M, ka->N, K,
                                                                    t / tiles_n, t % tiles_n, k_a << 8, (k_b - k_a) << 8,
                                                                    nullptr, mode, c, first, raise, defer);
  }
}

constexpr int kStreamKMaxGrid = 256;
constexpr int64_t kStreamKSlotBytes = 8 * 128 * 64 * 4;  // 256 x 256 fp32
constexpr int64_t kStreamKFlagBytes = 4096;
constexpr int kStreamKSpinLimit = 1 << 21;

template <bool W4, bool SWIGLU>
int launch_streamk(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y, int M, int N,
                   int K, void* ws, int64_t ws_bytes, int epoch, int spin_limit, int publish, hipStream_t stream) {
  if (ws_bytes < olmo355_gemm_streamk_workspace_bytes() || epoch == 0) return O355_EINVAL;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    return O355_ELAUNCH;
  const int grid = std::min(cus >= 8 ? (cus & ~7) : cus, kStreamKMaxGrid);
  if (grid <= 0) return O355_ELAUNCH;
  const int tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256;  // fused SwiGLU: 128 up + 128 gate columns per tile
  if ((int64_t)tiles_m * tiles_n * (K >> 8) < grid) return O355_EUNSUPPORTED;  // every workgroup must own at least one unit
  auto kern = gemm_streamk_kernel<2, 4, 4, 2, W4, SWIGLU>;
  const size_t lds = (size_t)(3 * 32 + 2 * 32) * 1024;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return O355_ELAUNCH;
  int* flags = reinterpret_cast<int*>(ws);
  float* slots = reinterpret_cast<float*>(reinterpret_cast<char*>(ws) + kStreamKFlagBytes);
  if ((int64_t)tiles_m * tiles_n * (K >> 8) * grid >= (1ll << 31)) return O355_EUNSUPPORTED;
  const StreamKArgs args{x, wt, st, zt, y, slots, flags, M, N, K, tiles_n, tiles_m * tiles_n, spin_limit, publish, epoch};
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), lds, stream, args);
  O355_CHECK_LAUNCH();
}

template <int WAVES_M, int WAVES_N, int WMT, int WNT, bool W4, bool SWIGLU = false, bool F16 = false>
int launch_gemm(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y, int M, int N,
                int K, hipStream_t stream) {
  constexpr int BM = 32 * WMT * WAVES_M, BN = 32 * WNT * WAVES_N;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;  // fused SwiGLU: N/2 divides by BN/2
  const size_t lds = (size_t)(3 * (BM / 8) + 2 * (BN / 8)) * 1024;
  auto kern = gemm_kernel<WAVES_M, WAVES_N, WMT, WNT, W4, SWIGLU, F16>;
  if (lds > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) !=
        hipSuccess)
      return O355_ELAUNCH;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n)), dim3(64 * WAVES_M * WAVES_N), lds, stream, x, wt, st, zt,
                     y, M, N, K, tiles_m, tiles_n);
  O355_CHECK_LAUNCH();
}

// Split-K plan for 128 x 64 tiles (two workgroups per CU), from measurements at N = 4096 .. 22016, K = 4096 and
// 11008, M = 96 .. 512: as many splits as keep the launch within two workgroups per CU and leave each at least
// 1024 of K (16 stages); with every CU already holding a tile a split pays only for long K (the two workgroups
// of a CU share its LDS bandwidth); 1 = do not split (for M <= 64: call the small-M entry).  K must divide into units of 256 and N into whole tiles.
int splitk_plan(int M, int N, int K) {
  if ((K & 255) || (N & 63) || ((int64_t)M * N & 3)) return 1;
  // 33 .. 64 rows belong to the staged-activation kernel except for narrow outputs over a long K (ff_out), where
  // 64 x 128 tiles split eight ways take 20 us against its 35 (N = 4096, K = 11008)
  if (M <= 64) return (M > 32 && (N & 127) == 0 && N <= 4096 && K >= 8192) ? 8 : 1;
  const int64_t tiles = (int64_t)((M + 127) / 128) * (N / 64);
  if (tiles > 256 || (tiles > 192 && K < 8192)) return 1;
  const int z = std::min(std::min((int)(512 / tiles), K / 1024), 16);
  return z < 2 ? 1 : z;
}

template <int WAVES_M, int WAVES_N, bool W4>
int launch_splitk_shape(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y, int M,
                        int N, int K, int splits, float* part, hipStream_t stream) {
  constexpr int BM = 32 * WAVES_M, BN = 32 * WAVES_N;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = N / BN;
  const size_t lds = (size_t)(3 * (BM / 8) + 2 * (BN / 8)) * 1024;
  auto kern = gemm_splitk_kernel<WAVES_M, WAVES_N, 1, 1, W4>;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) !=
      hipSuccess)
    return O355_ELAUNCH;
  hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n), (unsigned)splits), dim3(512), lds, stream, x, wt, st, zt,
                     part, M, N, K, tiles_m, tiles_n);
  const int64_t n4 = (int64_t)M * N / 4;
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, stream,
                     reinterpret_cast<const f32x4*>(part), reinterpret_cast<u32x2*>(y), n4, splits);
  O355_CHECK_LAUNCH();
}

// up to 64 rows: 64 x 128 tiles (no matrix-core work on rows that do not exist); otherwise 128 x 64
template <bool W4>
int launch_splitk(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y, int M, int N,
                  int K, int splits, float* part, hipStream_t stream) {
  if (M <= 64 && (N & 127) == 0) return launch_splitk_shape<2, 4, W4>(x, wt, st, zt, y, M, N, K, splits, part, stream);
  return launch_splitk_shape<4, 2, W4>(x, wt, st, zt, y, M, N, K, splits, part, stream);
}

// Tiles are 256 rows by 256, 192 or 128 columns, or 128 rows by 128 or 64 columns.  A launch runs in
// rounds of one tile per CU (two for the smallest tile, whose LDS fits twice), and the time of a round
// is far from proportional to the tile's area: a K-stage costs about 0.5 us of latency however small
// the tile.  The table holds measured microseconds per round at K = 4096 with int4 weights (the ratios
// are what matters); the shape with the smallest rounds x time wins.
template <bool W4, bool F16 = false>
int dispatch_gemm(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y, int M,
                  int N, int K, hipStream_t stream, int force_tile = 0) {  // force_tile: 1000 * rows + columns, 0 = choose
  const int cus = 256;
  struct Shape { int bm, bn, per_cu; double round_us; };
  static const Shape shapes[] = {{256, 256, 1, 95.}, {256, 192, 1, 80.}, {256, 128, 1, 55.}, {128, 128, 1, 37.}, {128, 64, 2, 47.}};
  int best = 0;
  double c = 1e300;
  for (const Shape& sh : shapes) {
    const int64_t tiles = (int64_t)((M + sh.bm - 1) / sh.bm) * ((N + sh.bn - 1) / sh.bn);
    const int64_t slots = cus * sh.per_cu;
    double ci = (double)((tiles + slots - 1) / slots) * sh.round_us;
    if (sh.per_cu == 2 && tiles <= cus) ci = 32.;  // one tile per CU: no sharing of the CU
    if (ci < c) c = ci, best = 1000 * sh.bm + sh.bn;
  }
  if (force_tile) best = force_tile < 1000 ? 256000 + force_tile : force_tile;
  switch (best) {
    case 256256: return launch_gemm<2, 4, 4, 2, W4, false, F16>(x, wt, st, zt, y, M, N, K, stream);
    case 256192: return launch_gemm<4, 2, 2, 3, W4, false, F16>(x, wt, st, zt, y, M, N, K, stream);
    case 256128: return launch_gemm<4, 2, 2, 2, W4, false, F16>(x, wt, st, zt, y, M, N, K, stream);
    case 128128: return launch_gemm<2, 4, 2, 1, W4, false, F16>(x, wt, st, zt, y, M, N, K, stream);
    case 128064: return launch_gemm<4, 2, 1, 1, W4, false, F16>(x, wt, st, zt, y, M, N, K, stream);
  }
  return O355_EINVAL;
}

}  // namespace

// the epilogues store 16 bytes at a time
static inline bool misaligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0; }

extern "C" int olmo355_w4_gemm_tile(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                                    uint16_t* y, int M, int N, int K, int tile, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0 || tile < 0) return O355_EINVAL;
  if (misaligned16(y)) return O355_EINVAL;
  if ((K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  return dispatch_gemm<true>(x, wt, st, zt, y, M, N, K, as_stream(stream), tile);
}

extern "C" int olmo355_b16_gemm_tile(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K, int tile,
                                     void* stream) {
  if (!x || !wt || !y || M <= 0 || N <= 0 || K <= 0 || tile < 0) return O355_EINVAL;
  if (misaligned16(y)) return O355_EINVAL;
  if ((K & 63) || (N & 15)) return O355_EUNSUPPORTED;
  return dispatch_gemm<false>(x, reinterpret_cast<const uint32_t*>(wt), nullptr, nullptr, y, M, N, K, as_stream(stream),
                              tile);
}

extern "C" int olmo355_w4_gemm(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                               uint16_t* y, int M, int N, int K, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (misaligned16(y)) return O355_EINVAL;
  if ((K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  return dispatch_gemm<true>(x, wt, st, zt, y, M, N, K, as_stream(stream));
}

// fp16 activations in, fp16 out; the weights dequantised to fp16 as the reference's QuantLinear does
// (qlinear_cuda_old.py:253-265,287-290).  Any M; tiled launches only (no split-K or stream-K form).
extern "C" int olmo355_w4_gemm_f16(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                                   uint16_t* y, int M, int N, int K, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (misaligned16(y)) return O355_EINVAL;
  if ((K & 127) || (N & 15)) return O355_EUNSUPPORTED;
  return dispatch_gemm<true, true>(x, wt, st, zt, y, M, N, K, as_stream(stream));
}

extern "C" int olmo355_gemm_splitk_plan(int M, int N, int K) { return splitk_plan(M, N, K); }

// ---- stream-K entries ------------------------------------------------------------------------------------
extern "C" int64_t olmo355_gemm_streamk_workspace_bytes(void) { return kStreamKFlagBytes + kStreamKMaxGrid * kStreamKSlotBytes; }

// 1 when the stream-K form is expected to beat the tiled launch.  Measured on the 7B shapes at 2048 rows: where the
// 256 x 256 tiles make a whole number of rounds the two are level; with 1.5 or 2.7 tiles per CU stream-K gains
// 4-15 %; with fewer tiles than CUs every tile is shared and the hand-over (about 15 us of partials written, read
// and waited for) must be earned by the better rate of the large tile: yes at K = 11008, no at K = 4096.  With a
// quarter to a half of the CUs' worth of tiles only a long K pays (1024 rows: N = 4096, K = 11008 94 against 111 us
// for the best tiled launch; N = K = 4096 51 against 44).
extern "C" int olmo355_gemm_streamk_plan(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0 || (K & 255) || (N & 15)) return 0;
  const int64_t tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
  if (tiles < 128) return tiles >= 64 && K >= 8192 ? 1 : 0;
  if (tiles < 256) return 2.0 * M * N * K >= 150e9 ? 1 : 0;
  const int64_t rounds = (tiles + 255) / 256;
  return tiles * 100 < rounds * 256 * 92 ? 1 : 0;  // the last round less than 92 % full
}

static int streamk_args_ok(const void* x, const void* wt, const void* y, const void* ws, int M, int N, int K) {
  if (!x || !wt || !y || !ws || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (misaligned16(y) || misaligned16(ws)) return O355_EINVAL;
  if ((K & 255) || (N & 15)) return O355_EUNSUPPORTED;
  return O355_OK;
}

extern "C" int olmo355_w4_gemm_streamk(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                                       uint16_t* y, int M, int N, int K, void* workspace, int64_t ws_bytes, int epoch, void* stream) {
  if (!st || !zt) return O355_EINVAL;
  if (const int rc = streamk_args_ok(x, wt, y, workspace, M, N, K)) return rc;
  return launch_streamk<true, false>(x, wt, st, zt, y, M, N, K, workspace, ws_bytes, epoch, kStreamKSpinLimit, 1, as_stream(stream));
}

extern "C" int olmo355_w4_gemm_swiglu_streamk(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                                              uint16_t* y, int M, int N, int K, void* workspace, int64_t ws_bytes, int epoch, void* stream) {
  if (!st || !zt) return O355_EINVAL;
  if (const int rc = streamk_args_ok(x, wt, y, workspace, M, N, K)) return rc;
  if ((N & 255) || (int64_t)(N >> 4) * (K >> 7) * 1024 >= (1ll << 32)) return O355_EUNSUPPORTED;
  return launch_streamk<true, true>(x, wt, st, zt, y, M, N, K, workspace, ws_bytes, epoch, kStreamKSpinLimit, 1, as_stream(stream));
}

extern "C" int olmo355_b16_gemm_streamk(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K,
                                        void* workspace, int64_t ws_bytes, int epoch, void* stream) {
  if (const int rc = streamk_args_ok(x, wt, y, workspace, M, N, K)) return rc;
  return launch_streamk<false, false>(x, reinterpret_cast<const uint32_t*>(wt), nullptr, nullptr, y, M, N, K, workspace,
                                      ws_bytes, epoch, kStreamKSpinLimit, 1, as_stream(stream));
}

// test hook: the finishing workgroups' patience and whether partials are announced at all
extern "C" int olmo355_w4_gemm_streamk_patience(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                                             uint16_t* y, int M, int N, int K, void* workspace, int64_t ws_bytes, int epoch,
                                             int spin_limit, int publish, void* stream) {
  if (!st || !zt || spin_limit < 0) return O355_EINVAL;
  if (const int rc = streamk_args_ok(x, wt, y, workspace, M, N, K)) return rc;
  return launch_streamk<true, false>(x, wt, st, zt, y, M, N, K, workspace, ws_bytes, epoch, spin_limit, publish, as_stream(stream));
}

extern "C" int olmo355_w4_gemm_splitk(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                                      uint16_t* y, int M, int N, int K, int splits, float* workspace, void* stream) {
  if (!x || !wt || !st || !zt || !y || !workspace || M <= 0 || N <= 0 || K <= 0 || splits < 2) return O355_EINVAL;
  if (misaligned16(workspace)) return O355_EINVAL;
  if ((K & 255) || (N & 63) || ((int64_t)M * N & 3) || splits > (K >> 8)) return O355_EUNSUPPORTED;
  return launch_splitk<true>(x, wt, st, zt, y, M, N, K, splits, workspace, as_stream(stream));
}

extern "C" int olmo355_b16_gemm_splitk(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K,
                                       int splits, float* workspace, void* stream) {
  if (!x || !wt || !y || !workspace || M <= 0 || N <= 0 || K <= 0 || splits < 2) return O355_EINVAL;
  if (misaligned16(workspace)) return O355_EINVAL;
  if ((K & 255) || (N & 63) || ((int64_t)M * N & 3) || splits > (K >> 8)) return O355_EUNSUPPORTED;
  return launch_splitk<false>(x, reinterpret_cast<const uint32_t*>(wt), nullptr, nullptr, y, M, N, K, splits, workspace,
                              as_stream(stream));
}

extern "C" int olmo355_w4_gemm_swiglu(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                                      uint16_t* y, int M, int N, int K, void* stream) {
  if (!x || !wt || !st || !zt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (misaligned16(y)) return O355_EINVAL;
  if ((K & 127) || (N & 255) || (int64_t)(N >> 4) * (K >> 7) * 1024 >= (1ll << 32)) return O355_EUNSUPPORTED;
  // rounds of one tile per CU, as in dispatch_gemm: 256 or 128 virtual columns (half up, half gate) per tile
  const int64_t tm = (M + 255) / 256;
  const double c256 = (double)((tm * (N / 256) + 255) / 256) * 95., c128 = (double)((tm * (N / 128) + 255) / 256) * 55.;
  if (c128 < c256) return launch_gemm<4, 2, 2, 2, true, true>(x, wt, st, zt, y, M, N, K, as_stream(stream));
  return launch_gemm<2, 4, 4, 2, true, true>(x, wt, st, zt, y, M, N, K, as_stream(stream));
}

extern "C" int olmo355_b16_gemm(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K,
                                void* stream) {
  if (!x || !wt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (misaligned16(y)) return O355_EINVAL;
  if ((K & 63) || (N & 15)) return O355_EUNSUPPORTED;
  return dispatch_gemm<false>(x, reinterpret_cast<const uint32_t*>(wt), nullptr, nullptr, y, M, N, K,
                              as_stream(stream));
}

// fp16 activations, dense fp16 weights in the tiled layout of olmo355_b16_repack (a 16-bit shuffle: either type), fp16
// out.  Any M; tiled launches only.
extern "C" int olmo355_f16_gemm(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K,
                                void* stream) {
  if (!x || !wt || !y || M <= 0 || N <= 0 || K <= 0) return O355_EINVAL;
  if (misaligned16(y)) return O355_EINVAL;
  if ((K & 63) || (N & 15)) return O355_EUNSUPPORTED;
  return dispatch_gemm<false, true>(x, reinterpret_cast<const uint32_t*>(wt), nullptr, nullptr, y, M, N, K,
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
