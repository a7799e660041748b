// Several int4 linears of a decode step in ONE launch (at most 4 rows): y_p = x_p . W_p for p = 0 .. n-1, where
// x_{p+1} is made from y_p (directly, or as resid + rmsnorm(y_p)), e.g. attn_out -> ff_proj -> ff_out -> the next
// block's att_proj (olmo/model.py:786-821 and :746-757 of the following block).
//
// Why one launch: a decode linear streams 9 .. 47 MB and lives for 4 .. 12 us, of which 3 .. 5 us are the launch
// boundary and the ramp of the first weight requests.  Weights do not depend on activations, so here the
// requests for phase p+1's weights go out *before* the workgroup waits for phase p to finish everywhere: the
// memory system keeps streaming during the hand-over.
//
// Shape of the kernel.  A persistent grid of one workgroup per CU (8 waves); all workgroups are resident, so a
// grid-wide barrier between phases cannot deadlock (and its wait is bounded anyway: on time-out a status word
// is set and the kernel runs to its end).  In phase p workgroup b owns the column tiles (16 columns; with the
// SwiGLU epilogue an up tile and its gate tile) b', b' + grid, ... with b' = (b + rot_p) mod grid.  The
// K dimension of a tile is cut into pieces of 4 groups of 128 rows (4 KiB of packed weights); the workgroup's
// (tile, piece) items are dealt round-robin to its waves, and a wave's items of all phases form ONE sequence
// that it requests in order into a private ring of LDS slots (memory -> LDS directly, no registers, no
// address arithmetic per lane), refilling a slot as soon as it has been consumed -- whatever phase the next
// item belongs to.  Loads of a wave complete in order, so "item j has landed" is one s_waitcnt on the number of
// requests issued after it.
// Every item is one accumulator pass of the "four groups share one MFMA accumulator" scheme of the small-M
// kernel (gemv.hip): group u of the piece puts the activations in operand rows 4u .. 4u+3, the lanes of row
// block u hold that group's scale and zero, acc += scale * (T - (128 + zero) * X), X from a ones-MFMA.  The
// activations of a phase are staged in LDS once per workgroup, each wave its share of the 512-element pieces, all
// requests of a wave in one batch: plain copy, or resid + rmsnorm(a) from the producer's per-tile sums of squares
// (olmo/model.py:241-255, same rounding points as elementwise.hip).  Partial sums meet in LDS; wave 0 adds them in wave order, rounds, applies SwiGLU
// (olmo/model.py:365-368) or leaves per-tile sums of squares, and publishes the rows with device-scope stores
// before it arrives at the barrier; consumers read them with device-scope loads (the L2 of another XCD may hold
// stale lines).
#include <algorithm>

#include "common.h"

namespace {

constexpr int kCW = 8;    // waves per workgroup
constexpr int kCT = 8;    // column tiles per workgroup and phase
constexpr int kCP = O355_CHAIN_MAX_PHASES;
constexpr int kPiece = 512;                       // activations per item: 4 groups of 128
constexpr int kSlotW = 4096, kSlotS = 256, kSlotZ = 256;  // every lane of a direct-to-LDS load writes its 4 bytes (zeros when out of range)
constexpr int kSlotBytes = kSlotW + kSlotS + kSlotZ;  // packed weights, their scales (window of 64 x 4 bytes), zeros
constexpr int kLoadsPerItem = 6;
constexpr int kMaxSlots = 3;
constexpr int kRedFloats = kCT * 64;              // per wave: [tile][4 rows][16 columns]
constexpr int kOob = (int)0xFFFFFF00u;            // buffer voffset beyond any resource: nothing is fetched
constexpr int kSc1 = 16;                          // cache policy: device-coherent access (bypasses a stale L2 line)

struct ChainArgs {
  olmo355_chain_phase ph[kCP];
  int n_phases, M, spin_limit, slots, xpieces;  // xpieces: 512-element pieces of the longest K
  int32_t* sync;    // [0]: epoch base; [64 .. 64 + grid): one arrival flag per workgroup (see olmo355_w4_chain_sync_ints)
  int32_t* status;  // set to 1 when a wait timed out
  int64_t* trace;   // NULL, or [grid][kCW][kCP][8] time stamps (100 MHz clock) of a tuning run
};

struct Plan {  // one phase as this workgroup sees it; every field is wave-uniform
  int G, QPT, ntiles, tpu, half, first, n_tiles, n_items;
};

__device__ __forceinline__ Plan make_plan(const olmo355_chain_phase& ph, int wg, int nwg) {
  Plan p;
  p.G = ph.K >> 7;
  p.QPT = (p.G + 3) >> 2;
  p.ntiles = ph.N >> 4;
  p.tpu = ph.swiglu ? 2 : 1;
  p.half = ph.swiglu ? (p.ntiles >> 1) : 0;
  const int units = ph.swiglu ? (p.ntiles >> 1) : p.ntiles;
  int first = wg + ph.rot;
  if (first >= nwg) first -= nwg;
  p.first = first;
  const int n_units = first < units ? (units - first + nwg - 1) / nwg : 0;
  p.n_tiles = n_units * p.tpu;
  p.n_items = p.n_tiles * p.QPT;
  return p;
}

// cursor over one wave's items of a phase: item ordinal k is workgroup item wave + kCW * k = (tile tl, piece q)
struct Cursor {
  int tl, q;
  __device__ __forceinline__ void start(const Plan& p, int wave) {
    tl = wave / p.QPT;
    q = wave - tl * p.QPT;
  }
  __device__ __forceinline__ void advance(const Plan& p) {
    q += kCW;
    while (q >= p.QPT) q -= p.QPT, ++tl;
  }
  __device__ __forceinline__ int tile(const Plan& p, int nwg) const {
    const int ul = p.tpu == 2 ? (tl >> 1) : tl, h = p.tpu == 2 ? (tl & 1) : 0;
    return p.first + ul * nwg + h * p.half;
  }
};

__device__ __forceinline__ void compiler_fence() { asm volatile("" ::: "memory"); }

template <typename T>
__device__ __forceinline__ void store_dev(T* p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// at most kLoadsPerItem * items vector-memory operations of this wave still outstanding (items beyond 3 count as 3)
__device__ __forceinline__ void wait_items_after(int items) {
  if (items <= 0) __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));
  else if (items == 1) __builtin_amdgcn_s_waitcnt(waitcnt_imm(kLoadsPerItem, false));
  else if (items == 2) __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * kLoadsPerItem, false));
  else __builtin_amdgcn_s_waitcnt(waitcnt_imm(3 * kLoadsPerItem, false));
}

__global__ __launch_bounds__(kCW * 64) void w4_chain_kernel(ChainArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int wg = blockIdx.x, nwg = gridDim.x, M = a.M, S = a.slots;
  const int xbytes = (a.xpieces * M + 1) * kPiece * 2;                          // [piece][row][512], then a zero row
  unsigned char* ring = smem + wave * (S * kSlotBytes);                         // this wave's weight slots
  unsigned char* xb = smem + kCW * S * kSlotBytes;                              // the phase's activations (whole workgroup)
  const int zero_off = a.xpieces * M * kPiece * 2;
  float* red = reinterpret_cast<float*>(smem + kCW * S * kSlotBytes + xbytes);  // [kCW][kCT][64]
  float* myred = red + wave * kRedFloats;

  // the zero row (operand rows that carry no activation row read it) and an empty reduction area
  if (wave == 0) *reinterpret_cast<u32x4*>(xb + zero_off + lane * 16) = u32x4{0u, 0u, 0u, 0u};
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < kRedFloats / 256; ++c) *reinterpret_cast<f32x4*>(myred + c * 256 + lane * 4) = zero4;

  // operand row `col` of group u is activation row col - 4u when that is in [0, M), else the zero row
  int rowsel[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int rel = col - 4 * u;
    rowsel[u] = (rel >= 0 && rel < M) ? rel : -1;
  }
  const UnpackConsts uc;
  const bf16x8 ones = ones_bf16x8();
  const int lane16 = lane * 16;

  // ---- the requesting side: a cursor that runs ahead of the computing side, across phase boundaries -------------
  int ip = 0, ileft = 0;  // phase of the next request, items of this wave left in it
  Plan iplan;
  Cursor icur;
  __amdgpu_buffer_rsrc_t irw, irs, irz;
  int issued = 0, consumed = 0;
  auto enter_phase = [&]() {  // position the cursor on this wave's first item of phase ip, skipping phases without one
    while (ip < a.n_phases) {
      iplan = make_plan(a.ph[ip], wg, nwg);
      ileft = iplan.n_items > wave ? (iplan.n_items - wave + kCW - 1) / kCW : 0;
      if (ileft > 0) {
        const int total = iplan.ntiles * iplan.G;
        irw = make_rsrc(a.ph[ip].wt, (int64_t)total * 1024);
        irs = make_rsrc(a.ph[ip].st, (int64_t)total * 32);
        irz = make_rsrc(a.ph[ip].zt, (int64_t)total * 8);
        icur.start(iplan, wave);
        return;
      }
      ++ip;
    }
  };
  // Wave 0 publishes the rows and polls the barrier, and both must not queue behind its own weight requests
  // (a wave's memory operations complete in order): it only asks for weights of phases whose barrier it has passed.
  auto issue_next = [&](int last_phase) {
    if (ip >= a.n_phases || ip > last_phase) return;
    unsigned char* sl = ring + (issued % S) * kSlotBytes;
    const int G = iplan.G, tg = icur.tile(iplan, nwg) * G, g0 = 4 * icur.q;
#pragma unroll
    for (int u = 0; u < 4; ++u)  // past the end of K: any valid group, its scale is forced to zero
      __builtin_amdgcn_raw_ptr_buffer_load_lds(irw, (lds_ptr_t)(sl + u * 1024), 16, lane16, (tg + min(g0 + u, G - 1)) * 1024, 0, 2);
    // scales: 32 bytes per group (8 lanes of 4 bytes), zeros: 8 bytes per group (2 lanes); groups past K are not fetched
    const int sv = (lane < 32 && g0 + (lane >> 3) < G) ? lane * 4 : kOob;
    const int zv = (lane < 8 && g0 + (lane >> 1) < G) ? lane * 4 : kOob;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(irs, (lds_ptr_t)(sl + kSlotW), 4, sv, (tg + g0) * 32, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(irz, (lds_ptr_t)(sl + kSlotW + kSlotS), 4, zv, (tg + g0) * 8, 0, 0);
    ++issued;
    if (--ileft > 0) {
      icur.advance(iplan);
    } else {
      ++ip;
      enter_phase();
    }
  };
  enter_phase();
  for (int s = 0; s < S; ++s) issue_next(wave == 0 ? 0 : kCP);

  // time stamps of a tuning run: 0 phase entered, 1 activations staged, 2 staging barrier passed, 3 first item landed,
  // 4 items done, 5 rows published (wave 0), 6 every workgroup arrived (wave 0), 7 phase left
  auto stamp = [&](int p, int ev) {
    if (a.trace && lane == 0) a.trace[((wg * kCW + wave) * kCP + p) * 8 + ev] = (int64_t)__builtin_amdgcn_s_memrealtime();
  };
  bool failed = false;
  const int epoch_base = a.n_phases > 1 ? __hip_atomic_load(a.sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
  for (int p = 0; p < a.n_phases; ++p) {
    const olmo355_chain_phase& ph = a.ph[p];
    const Plan plan = make_plan(ph, wg, nwg);
    const int K = ph.K;
    const bool chained = ph.resid != nullptr;
    const bool writer = chained && plan.first == 0;  // the workgroup that owns tile 0 also writes x_out
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(ph.x, (int64_t)M * K * 2);
    const __amdgpu_buffer_rsrc_t rr = make_rsrc(ph.resid, chained ? (int64_t)M * K * 2 : 0);
    const __amdgpu_buffer_rsrc_t rn = make_rsrc(ph.norm_w, chained ? (int64_t)K * 2 : 0);
    const __amdgpu_buffer_rsrc_t ro = make_rsrc(ph.x_out, chained ? (int64_t)M * K * 2 : 0);
    const int my_items = plan.n_items > wave ? (plan.n_items - wave + kCW - 1) / kCW : 0;

    const int issued_before_stage = issued;
    stamp(p, 0);
    // ---- stage the phase's activations: wave w takes the pieces w, w + 8, ... of every row; one batch of requests
    // for the sums of squares, the norm weight and row 0, one more batch per further row -------------------------------
    {
      const int n_ssq = K >> 4;
      f32x4 pv[4][4];
      u32x4 nv[4];
      bool plive[4];
      int pvo[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int q = wave + kCW * i;
        plive[i] = q < plan.QPT && q * kPiece + lane * 8 < K;
        pvo[i] = plive[i] ? lane16 + q * kPiece * 2 : kOob;
      }
      if (chained) {
#pragma unroll
        for (int m = 0; m < 4; ++m)
          if (m < M) {
            const __amdgpu_buffer_rsrc_t rp = make_rsrc(ph.ssq_in + (int64_t)m * n_ssq, (int64_t)n_ssq * 4);
#pragma unroll
            for (int c = 0; c < 4; ++c)
              pv[m][c] = c * 256 < n_ssq ? __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rp, lane16 + c * 1024, 0, kSc1)) : zero4;
          }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (wave + kCW * i < plan.QPT) nv[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rn, pvo[i], 0, 0));
      }
      float rstd[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
      for (int m = 0; m < M; ++m) {
        {
          u32x4 av[4], rv[4];
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (wave + kCW * i < plan.QPT) {
              av[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, pvo[i], m * K * 2, kSc1));
              if (chained) rv[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rr, pvo[i], m * K * 2, kSc1));
            }
          if (m == 0 && chained) {  // 1 / rms of every row (fixed order: the same in every wave of every workgroup)
#pragma unroll
            for (int mm = 0; mm < 4; ++mm)
              if (mm < M) {
                float ss = (pv[mm][0][0] + pv[mm][0][1]) + (pv[mm][0][2] + pv[mm][0][3]);
#pragma unroll
                for (int c = 1; c < 4; ++c) ss += (pv[mm][c][0] + pv[mm][c][1]) + (pv[mm][c][2] + pv[mm][c][3]);
                ss = wave_sum_dpp(ss);
                rstd[mm] = 1.f / sqrtf(ss / (float)K + ph.eps);
              }
          }
          const float rs = m == 0 ? rstd[0] : (m == 1 ? rstd[1] : (m == 2 ? rstd[2] : rstd[3]));
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int q = wave + kCW * i;
            if (q < plan.QPT) {
              u32x4 o = av[i];
              if (chained) {
                float f[8], r[8], w[8];
                unpack8(av[i], f);
                unpack8(rv[i], r);
                unpack8(nv[i], w);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  const float y0 = round_bf16(w[2 * e] * round_bf16(f[2 * e] * rs));
                  const float y1 = round_bf16(w[2 * e + 1] * round_bf16(f[2 * e + 1] * rs));
                  o[e] = pack_bf16x2(r[2 * e] + y0, r[2 * e + 1] + y1);
                }
                if (writer && plive[i]) __builtin_amdgcn_raw_buffer_store_b128(o, ro, pvo[i], m * K * 2, kSc1);
              }
              if (!plive[i]) o = u32x4{0u, 0u, 0u, 0u};
              *reinterpret_cast<u32x4*>(xb + (q * M + m) * (kPiece * 2) + lane16) = o;
            }
          }
        }
      }
    }
    stamp(p, 1);
    lds_barrier();
    stamp(p, 2);

    // ---- this wave's items of the phase ----------------------------------------------------------------------------
    Cursor cur;
    cur.start(plan, wave);
    int cur_q = -1, cur_tl = -1;
    f32x4 acc = zero4, xsum = zero4;
    bf16x8 af[4][4];
    auto flush = [&](int tl) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = acc[r];
        v = combine_xor16(v, AddOp{});
        v = combine_xor32(v, AddOp{});
        if (kq == 0) myred[tl * 64 + r * 16 + col] = v;
      }
    };
    for (int k = 0; k < my_items; ++k) {
      if (cur.q != cur_q) {  // operand fragments of piece q, and the sums of its groups on the matrix cores
        cur_q = cur.q;
        xsum = zero4;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int base = (rowsel[u] >= 0 ? (cur.q * M + rowsel[u]) * (kPiece * 2) : zero_off) + (128 * u + 8 * kq) * 2;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            af[u][j] = *reinterpret_cast<const bf16x8*>(xb + base + 64 * j);
            xsum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[u][j], ones, xsum, 0, 0, 0);
          }
        }
      }
      if (cur.tl != cur_tl) {
        if (cur_tl >= 0) flush(cur_tl);
    stamp(p, 4);
        cur_tl = cur.tl;
        acc = zero4;
      }
      // ---- the oldest request of the ring is this item ---------------------------------------------------------------
      wait_items_after(issued - consumed - 1);
      compiler_fence();
      if (k == 0) stamp(p, 3);
      const unsigned char* sl = ring + (consumed % S) * kSlotBytes;
      u32x4 w[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) w[u] = *reinterpret_cast<const u32x4*>(sl + u * 1024 + lane16);
      const uint32_t s16 = *reinterpret_cast<const uint16_t*>(sl + kSlotW + kq * 32 + col * 2);
      const uint32_t z8 = *(sl + kSlotW + kSlotS + kq * 8 + (col >> 1));
      f32x4 t0 = zero4, t1 = zero4;
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
          t0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[u][j], unpack_w4_bias128(w[u][j], uc), t0, 0, 0, 0);
          t1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[u][j + 1], unpack_w4_bias128(w[u][j + 1], uc), t1, 0, 0, 0);
        }
      const float sc = (4 * cur.q + kq < plan.G) ? (float)__builtin_bit_cast(_Float16, (uint16_t)s16) : 0.f;
      const float nzc = -(float)(129 + (int)((z8 >> (4 * (col & 1))) & 15u));  // -(128 + (stored + 1))
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] = __builtin_fmaf(sc, __builtin_fmaf(nzc, xsum[r], t0[r] + t1[r]), acc[r]);
      ++consumed;
      compiler_fence();
      issue_next(wave == 0 ? p : kCP);  // the slot is free again: the next request of the sequence, of this phase or a later one
      cur.advance(plan);
    }
    if (cur_tl >= 0) flush(cur_tl);
    stamp(p, 4);
    // this wave's x_out stores have been acknowledged once only requests issued after them are outstanding
    if (writer) wait_items_after(min(issued - consumed, issued - issued_before_stage));

    // ---- hand-over: wave 0 publishes the rows, arrives and waits for every workgroup; the others sleep at the
    // workgroup barrier.  Requests for the next phases' weights are already in flight. ----------------------------------
    const bool more = p + 1 < a.n_phases;
    lds_barrier();
    if (wave == 0) {
      const int m = lane >> 4;
      const bool rowlive = m < M;
      for (int tl = 0; tl < plan.n_tiles; tl += plan.tpu) {
        const int ul = plan.tpu == 2 ? (tl >> 1) : tl;
        const int tile = plan.first + ul * nwg;
        float v0 = 0.f, v1 = 0.f;
#pragma unroll
        for (int w = 0; w < kCW; ++w) v0 += red[w * kRedFloats + tl * 64 + lane];
        if (plan.tpu == 2) {
#pragma unroll
          for (int w = 0; w < kCW; ++w) v1 += red[w * kRedFloats + (tl + 1) * 64 + lane];
        }
        float outv;
        int ncols;
        if (plan.tpu == 2) {  // SwiGLU: v0 = up, v1 = gate, each rounded as the Linear's bf16 output
          const float up = round_bf16(v0), gate = round_bf16(v1);
          const float sg = round_bf16(gate / (1.f + expf(-gate)));
          outv = round_bf16(sg * up);
          ncols = ph.N >> 1;
        } else {
          outv = round_bf16(v0);
          ncols = ph.N;
        }
        const uint32_t bits = f32_to_bf16_bits(outv);
        const uint32_t nb = __shfl_xor(bits, 1, 64);
        if (rowlive && (col & 1) == 0)
          store_dev(reinterpret_cast<uint32_t*>(ph.y + (int64_t)m * ncols + tile * 16 + col), bits | (nb << 16));
        if (ph.ssq_out) {
          const float q = row16_sum(outv * outv);
          if (rowlive && col == 0) store_dev(ph.ssq_out + (int64_t)m * plan.ntiles + tile, q);
        }
      }
      if (more) {
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));  // the rows have landed
        compiler_fence();
        stamp(p, 5);
        // Arrival: every workgroup owns one flag word and stores the barrier's epoch into it (no read-modify-write: 256
        // atomic adds on one address queue up for microseconds).  Epochs grow from launch to launch (the base lives in
        // sync[0]), so the flags never need clearing.  Waiting: one 16-byte load per lane reads 256 flags at once.
        const int epoch = epoch_base + p + 1;
        if (lane == 0) store_dev(a.sync + 64 + wg, epoch);
        if (!failed) {
          int spins = 0;
          for (;;) {
            bool all = true;
            for (int f0 = 0; f0 < nwg; f0 += 256) {
              const __amdgpu_buffer_rsrc_t rf = make_rsrc(a.sync + 64 + f0, (int64_t)min(nwg - f0, 256) * 4);
              const u32x4 fv = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rf, lane16, 0, kSc1));
              bool ok = true;
#pragma unroll
              for (int e = 0; e < 4; ++e) ok = ok && (f0 + lane * 4 + e >= nwg || (int)(fv[e] - (uint32_t)epoch) >= 0);
              all = all && __builtin_amdgcn_ballot_w64(!ok) == 0;
            }
            if (all) break;
            if (++spins > a.spin_limit) {
              failed = true;
              if (lane == 0) store_dev(a.status, (int32_t)1);
              break;
            }
            __builtin_amdgcn_s_sleep(1);
          }
        }
        compiler_fence();
      }
    }
    if (wave == 0) stamp(p, 6);
    lds_barrier();
    compiler_fence();
    stamp(p, 7);
    if (wave == 0 && more)
      for (int s = 0; s < S; ++s) issue_next(p + 1);  // its ring is empty: the first requests of the next phase
    // the reduction area is free again (wave 0 has read it): empty it for the next phase
#pragma unroll
    for (int c = 0; c < kRedFloats / 256; ++c) *reinterpret_cast<f32x4*>(myred + c * 256 + lane * 4) = zero4;
  }

  // ---- the next launch starts its epochs after this one's.  Workgroup 0 has passed a barrier by now, so every
  // workgroup has read the old base.
  if (wg == 0 && tid == 0 && a.n_phases > 1) store_dev(a.sync, epoch_base + a.n_phases - 1);
}

}  // namespace

extern "C" int olmo355_w4_chain_sync_ints(void) { return 64 + olmo355_w4_chain_grid(); }

extern "C" int olmo355_w4_chain_grid(void) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return 0;
  return cus;
}

extern "C" int olmo355_w4_chain_trace(const olmo355_chain_phase* phases, int n_phases, int M, int32_t* sync,
                                      int32_t* status, int spin_limit, int64_t* trace, void* stream) {
  if (!phases || !sync || !status || n_phases < 1 || n_phases > kCP || M < 1 || spin_limit < 1) return O355_EINVAL;
  if (M > 4) return O355_EUNSUPPORTED;
  const int grid = olmo355_w4_chain_grid();
  if (grid <= 0) return O355_ELAUNCH;
  ChainArgs a;
  for (int p = 0; p < n_phases; ++p) {
    const olmo355_chain_phase& ph = phases[p];
    if (!ph.x || !ph.wt || !ph.st || !ph.zt || !ph.y || ph.N <= 0 || ph.K <= 0) return O355_EINVAL;
    if ((ph.resid != nullptr) != (ph.ssq_in != nullptr) || (ph.resid && (!ph.norm_w || !ph.x_out))) return O355_EINVAL;
    if (ph.rot < 0 || ph.rot >= grid) return O355_EINVAL;
    if ((ph.K & 127) || (ph.N & (ph.swiglu ? 31 : 15)) || (ph.swiglu && ph.ssq_out)) return O355_EUNSUPPORTED;
    if ((ph.K >> 4) > 1024 || (int64_t)(ph.N >> 4) * (ph.K >> 7) * 1024 >= (1ll << 31)) return O355_EUNSUPPORTED;
    const int units = ph.swiglu ? (ph.N >> 5) : (ph.N >> 4);
    if (((units + grid - 1) / grid) * (ph.swiglu ? 2 : 1) > kCT) return O355_EUNSUPPORTED;
    a.ph[p] = ph;
  }
  a.n_phases = n_phases, a.M = M, a.spin_limit = spin_limit, a.sync = sync, a.status = status, a.trace = trace;
  int maxk = 0;
  for (int p = 0; p < n_phases; ++p) maxk = std::max(maxk, phases[p].K);
  a.xpieces = (maxk + kPiece - 1) / kPiece;
  // LDS: the phase's activations (+ a zero row), the reduction area, and as many weight slots per wave as still fit
  // (at most 3); always more than half of a CU's 160 KiB, so that exactly one workgroup lives on a CU
  const int fixed = (a.xpieces * M + 1) * kPiece * 2 + kCW * kRedFloats * 4;
  a.slots = std::min(kMaxSlots, (160 * 1024 - fixed) / (kCW * kSlotBytes));
  if (a.slots < 1) return O355_EUNSUPPORTED;
  if (a.slots < 2) a.slots = 1;
  const int lds = std::max(kCW * a.slots * kSlotBytes + fixed, 96 * 1024);
  auto kern = w4_chain_kernel;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
    return O355_ELAUNCH;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kCW * 64), lds, as_stream(stream), a);
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_w4_chain(const olmo355_chain_phase* phases, int n_phases, int M, int32_t* sync, int32_t* status,
                                int spin_limit, void* stream) {
  return olmo355_w4_chain_trace(phases, n_phases, M, sync, status, spin_limit, nullptr, stream);
}
