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
// (tile, piece) items are dealt round-robin to its waves.  A wave keeps up to 6 items in flight in registers;
// every item is one accumulator pass of the "four groups share one MFMA accumulator" scheme of the small-M
// kernel (gemv.hip): group u of the piece puts the activations in operand rows 4u .. 4u+3, the lanes of row
// block u hold that group's scale and zero, acc += scale * (T - (128 + zero) * X).  Each wave stages the 512
// activations of its piece itself (own LDS buffer, no workgroup barrier): plain copy, or resid + rmsnorm(a) from
// the producer's per-tile sums of squares (olmo/model.py:241-255, same rounding points as elementwise.hip).
// Partial sums meet in LDS; wave 0 adds them in wave order, rounds, applies SwiGLU (olmo/model.py:365-368) or
// leaves per-tile sums of squares, and publishes the rows with device-scope stores before it arrives at the
// barrier; consumers read them with device-scope loads (the L2 of another XCD may hold stale lines).
#include "common.h"

namespace {

constexpr int kCW = 8;    // waves per workgroup
constexpr int kCI = 6;    // items (4 KiB weight pieces) per wave held in registers
constexpr int kCT = 8;    // column tiles per workgroup and phase
constexpr int kCP = O355_CHAIN_MAX_PHASES;
constexpr int kPiece = 512;                       // activations per item: 4 groups of 128
constexpr int kXBytes = 5 * kPiece * 2;           // per wave: 4 rows + a zero row
constexpr int kRedFloats = kCT * 64;              // per wave: [tile][4 rows][16 columns]
constexpr int kChainLds = 96 * 1024;              // more than half a CU's LDS: exactly one workgroup per CU
constexpr int kOob = (int)0xFFFFFF00u;            // buffer voffset beyond any resource: the load returns zero
constexpr int kSc1 = 16;                          // cache policy: device-coherent access (bypasses a stale L2 line)

struct ChainArgs {
  olmo355_chain_phase ph[kCP];
  int n_phases, M, spin_limit;
  int32_t* sync;    // [n_phases + 1], zero on entry and on exit
  int32_t* status;  // set to 1 when a wait timed out
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

struct Item {
  int tile, tl, q;
  bool valid;
};

__device__ __forceinline__ Item item_of(const Plan& p, int i, int nwg) {
  Item it;
  it.valid = i < p.n_items;
  const int ic = it.valid ? i : 0;
  it.tl = ic / p.QPT;
  it.q = ic - it.tl * p.QPT;
  const int ul = p.tpu == 2 ? (it.tl >> 1) : it.tl, h = p.tpu == 2 ? (it.tl & 1) : 0;
  it.tile = p.first + ul * nwg + h * p.half;
  return it;
}

struct Slot {
  u32x4 w[4];
  uint32_t s16, z8;
};

// requests of one item; an invalid item asks beyond the resources (no traffic, zeros come back in order)
__device__ __forceinline__ void issue(Slot& s, const olmo355_chain_phase& ph, const Plan& p, const Item& it, int lane) {
  const int col = lane & 15, kq = lane >> 4;
  const int total = p.ntiles * p.G;
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(ph.wt, (int64_t)total * 1024);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(ph.st, (int64_t)total * 32);
  const __amdgpu_buffer_rsrc_t rz = make_rsrc(ph.zt, (int64_t)total * 8);
  const int tg = it.tile * p.G;
  const int wvoff = it.valid ? lane * 16 : kOob;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int g = min(4 * it.q + u, p.G - 1);  // past the end of K: any valid group, its scale is forced to zero
    s.w[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, wvoff, it.valid ? (tg + g) * 1024 : 0, 2));
  }
  const int gl = tg + min(4 * it.q + kq, p.G - 1);
  s.s16 = __builtin_amdgcn_raw_buffer_load_b16(rs, it.valid ? (gl * 16 + col) * 2 : kOob, 0, 0);
  s.z8 = __builtin_amdgcn_raw_buffer_load_b8(rz, it.valid ? gl * 8 + (col >> 1) : kOob, 0, 0);
}

__device__ __forceinline__ void compiler_fence() { asm volatile("" ::: "memory"); }

template <typename T>
__device__ __forceinline__ void store_dev(T* p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__global__ __launch_bounds__(kCW * 64) void w4_chain_kernel(ChainArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int wg = blockIdx.x, nwg = gridDim.x, M = a.M;
  unsigned char* xb = smem + wave * kXBytes;                                  // this wave's activations [M + 1][512]
  float* xs = reinterpret_cast<float*>(smem + kCW * kXBytes) + wave * 16;     // their sums per group: [4 groups][4 rows]
  float* red = reinterpret_cast<float*>(smem + kCW * kXBytes + kCW * 64);     // [kCW][kCT][64]
  float* myred = red + wave * kRedFloats;

  // the zero row (operand rows that carry no activation row read it) and an empty reduction area
  *reinterpret_cast<u32x4*>(xb + 4 * kPiece * 2 + lane * 16) = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
  for (int c = 0; c < kRedFloats / 256; ++c) *reinterpret_cast<f32x4*>(myred + c * 256 + lane * 4) = f32x4{0.f, 0.f, 0.f, 0.f};

  // operand row `col` of group u is activation row col - 4u when that is in [0, M), else the zero row
  int xoff[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int rel = col - 4 * u;
    xoff[u] = (((rel >= 0 && rel < M) ? rel : 4) * kPiece + 128 * u + 8 * kq) * 2;
  }
  const UnpackConsts uc;
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

  Slot slot[kCI];
  Plan plan = make_plan(a.ph[0], wg, nwg);
#pragma unroll
  for (int s = 0; s < kCI; ++s) issue(slot[s], a.ph[0], plan, item_of(plan, wave + kCW * s, nwg), lane);

  bool failed = false;
  for (int p = 0; p < a.n_phases; ++p) {
    const olmo355_chain_phase& ph = a.ph[p];
    const int K = ph.K;
    const bool chained = ph.resid != nullptr;
    const bool writer = chained && plan.first == 0;  // the workgroup that owns tile 0 also writes x_out
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(ph.x, (int64_t)M * K * 2);
    const __amdgpu_buffer_rsrc_t rr = make_rsrc(ph.resid, chained ? (int64_t)M * K * 2 : 0);
    const __amdgpu_buffer_rsrc_t rn = make_rsrc(ph.norm_w, chained ? (int64_t)K * 2 : 0);
    const __amdgpu_buffer_rsrc_t ro = make_rsrc(ph.x_out, chained ? (int64_t)M * K * 2 : 0);

    // ---- 1 / rms of every row, from the producer's per-tile sums of squares (fixed order: the same in every wave) ----
    float rstd[4] = {0.f, 0.f, 0.f, 0.f};
    const int my_items = plan.n_items > wave ? (plan.n_items - wave + kCW - 1) / kCW : 0;
    if (chained && my_items > 0) {
      const int n_ssq = K >> 4;
      f32x4 pv[4][4];
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const __amdgpu_buffer_rsrc_t rp = make_rsrc(ph.ssq_in + (int64_t)min(m, M - 1) * n_ssq, (int64_t)n_ssq * 4);
#pragma unroll
        for (int c = 0; c < 4; ++c)
          pv[m][c] = (m < M && c * 256 < n_ssq)
                         ? __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rp, lane * 16 + c * 1024, 0, kSc1))
                         : zero4;
      }
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        float ss = (pv[m][0][0] + pv[m][0][1]) + (pv[m][0][2] + pv[m][0][3]);
#pragma unroll
        for (int c = 1; c < 4; ++c) ss += (pv[m][c][0] + pv[m][c][1]) + (pv[m][c][2] + pv[m][c][3]);
        ss = wave_sum_dpp(ss);
        rstd[m] = 1.f / sqrtf(ss / (float)K + ph.eps);
      }
    }

    // ---- this wave's items: weights are in flight (or here), activations staged per piece --------------------------
    int cur_q = -1, cur_tl = -1;
    f32x4 acc = zero4, xsum = zero4;
    bf16x8 af[4][4];
    auto flush = [&](int tl) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = acc[r];
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        if (kq == 0) myred[tl * 64 + r * 16 + col] = v;
      }
    };
    const int rounds = (my_items + kCI - 1) / kCI;
    for (int round = 0; round < rounds; ++round) {
#pragma unroll
      for (int s = 0; s < kCI; ++s) {
        const int k = round * kCI + s;
        const Item it = item_of(plan, wave + kCW * k, nwg);
        if (it.valid) {  // wave-uniform
          if (it.q != cur_q) {
            // ---- stage the 512 activations of piece q for every row; their sums per group ------------------------
            cur_q = it.q;
            const int k0 = it.q * kPiece + lane * 8;
            const bool live = k0 < K;
            u32x4 nv = u32x4{0u, 0u, 0u, 0u};
            if (chained) nv = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rn, live ? lane * 16 : kOob, live ? it.q * kPiece * 2 : 0, 0));
            u32x4 av[4], rv[4];
#pragma unroll
            for (int m = 0; m < 4; ++m) {
              av[m] = rv[m] = u32x4{0u, 0u, 0u, 0u};
              if (m < M) {
                const int so = live ? (m * K + it.q * kPiece) * 2 : 0, vo = live ? lane * 16 : kOob;
                av[m] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, vo, so, kSc1));
                if (chained) rv[m] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rr, vo, so, kSc1));
              }
            }
            float sum4[4];
#pragma unroll
            for (int m = 0; m < 4; ++m) {
              u32x4 o = av[m];
              if (chained) {
                float f[8], r[8], w[8];
                unpack8(av[m], f);
                unpack8(rv[m], r);
                unpack8(nv, w);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  const float y0 = round_bf16(w[2 * e] * round_bf16(f[2 * e] * rstd[m]));
                  const float y1 = round_bf16(w[2 * e + 1] * round_bf16(f[2 * e + 1] * rstd[m]));
                  o[e] = pack_bf16x2(r[2 * e] + y0, r[2 * e + 1] + y1);
                }
                if (!live || m >= M) o = u32x4{0u, 0u, 0u, 0u};
                if (writer && live && m < M)
                  __builtin_amdgcn_raw_buffer_store_b128(o, ro, lane * 16, (m * K + it.q * kPiece) * 2, kSc1);
              }
              float g[8], sm = 0.f;
              unpack8(o, g);
#pragma unroll
              for (int e = 0; e < 8; ++e) sm += g[e];
              sum4[m] = row16_sum(sm);  // the 16 lanes of a row hold one group of 128
              if (m < M) *reinterpret_cast<u32x4*>(xb + m * kPiece * 2 + lane * 16) = o;
            }
            if (col == 0) *reinterpret_cast<f32x4*>(xs + kq * 4) = f32x4{sum4[0], sum4[1], sum4[2], sum4[3]};
            __builtin_amdgcn_wave_barrier();
            xsum = *reinterpret_cast<const f32x4*>(xs + kq * 4);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
              for (int j = 0; j < 4; ++j) af[u][j] = *reinterpret_cast<const bf16x8*>(xb + xoff[u] + 64 * j);
          }
          if (it.tl != cur_tl) {
            if (cur_tl >= 0) flush(cur_tl);
            cur_tl = it.tl;
            acc = zero4;
          }
          f32x4 t = zero4;
#pragma unroll
          for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int j = 0; j < 4; ++j)
              t = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[u][j], unpack_w4_bias128(slot[s].w[u][j], uc), t, 0, 0, 0);
          const float sc = (4 * it.q + kq < plan.G) ? (float)__builtin_bit_cast(_Float16, (uint16_t)slot[s].s16) : 0.f;
          const float nzc = -(float)(129 + (int)((slot[s].z8 >> (4 * (col & 1))) & 15u));  // -(128 + (stored + 1))
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[r] = __builtin_fmaf(sc, __builtin_fmaf(nzc, xsum[r], t[r]), acc[r]);
        }
        // refill the slot with a later item of this phase, if there is one
        if (round + 1 < rounds) issue(slot[s], ph, plan, item_of(plan, wave + kCW * (k + kCI), nwg), lane);
      }
    }
    if (cur_tl >= 0) flush(cur_tl);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, false));  // this wave's x_out stores have been acknowledged

    // ---- hand-over: the other waves ask for the next phase's weights at once and sleep at the barrier; wave 0
    // publishes the rows, arrives, waits for every workgroup, and only then asks for its own weights (its wait
    // must not queue behind them) ------------------------------------------------------------------------------------
    const bool more = p + 1 < a.n_phases;
    Plan next = plan;
    if (more) next = make_plan(a.ph[p + 1], wg, nwg);
    if (more && wave != 0) {
#pragma unroll
      for (int s = 0; s < kCI; ++s) issue(slot[s], a.ph[p + 1], next, item_of(next, wave + kCW * s, nwg), lane);
    }
    lds_barrier();
    if (wave == 0) {
      const int r = lane >> 4, m = r;
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
        if (lane == 0) __hip_atomic_fetch_add(a.sync + p, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (!failed) {
          int spins = 0;
          while (__hip_atomic_load(a.sync + p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < nwg) {
            if (++spins > a.spin_limit) {
              failed = true;
              if (lane == 0) store_dev(a.status, (int32_t)1);
              break;
            }
            __builtin_amdgcn_s_sleep(2);
          }
        }
        compiler_fence();
#pragma unroll
        for (int s = 0; s < kCI; ++s) issue(slot[s], a.ph[p + 1], next, item_of(next, wave + kCW * s, nwg), lane);
      }
    }
    lds_barrier();
    compiler_fence();
    // the reduction area is free again (wave 0 has read it): empty it for the next phase
#pragma unroll
    for (int c = 0; c < kRedFloats / 256; ++c) *reinterpret_cast<f32x4*>(myred + c * 256 + lane * 4) = zero4;
    plan = next;
  }

  // ---- leave the barrier counters at zero: the last workgroup to get here clears them ----------------------------
  if (tid == 0) {
    const int t = __hip_atomic_fetch_add(a.sync + a.n_phases, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (t == nwg - 1)
      for (int i = 0; i <= a.n_phases; ++i) store_dev(a.sync + i, (int32_t)0);
  }
}

}  // namespace

extern "C" int olmo355_w4_chain_grid(void) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return 0;
  return cus;
}

extern "C" int olmo355_w4_chain(const olmo355_chain_phase* phases, int n_phases, int M, int32_t* sync, int32_t* status,
                                int spin_limit, void* stream) {
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
  a.n_phases = n_phases, a.M = M, a.spin_limit = spin_limit, a.sync = sync, a.status = status;
  auto kern = w4_chain_kernel;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kChainLds) != hipSuccess)
    return O355_ELAUNCH;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kCW * 64), kChainLds, as_stream(stream), a);
  O355_CHECK_LAUNCH();
}
