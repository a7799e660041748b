// Two measuring probes, not part of the forward pass: what this GPU gives a kernel that only streams bytes
// from HBM, and one that only issues bf16 MFMAs on random operands.  bench.py reports them beside the
// achieved figures so that "fraction of the published peak" can be read against what is reachable at the
// same launch sizes on the same box.
#include "common.h"
#include "../../include/olmo355_debug.h"

namespace {

// Every wave reads 1 KiB pieces (16 bytes per lane, non-temporal) round-robin with U requests in flight and
// folds them into one word; nothing is written unless the fold hits a value it cannot predict.
template <int U>
__global__ __launch_bounds__(512) void stream_read_kernel(const u32x4* __restrict__ src, int64_t pieces,
                                                          uint32_t* __restrict__ sink) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 6), nw = (int64_t)gridDim.x * 8;
  uint32_t acc = 0;
  for (int64_t p = wave; p < pieces; p += nw * U) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t q = p + u * nw;
      v[u] = q < pieces ? __builtin_nontemporal_load(&src[q * 64 + lane]) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (acc == 0x9e3779b9u) sink[threadIdx.x] = acc;
}

// The same for many buffers in ONE launch of a grid that stays (two workgroups per CU): the pieces of all buffers
// form one sequence dealt round-robin to the waves, 8 requests in flight per wave at all times.  No launch
// boundary, no ramp per buffer: what the memory system sustains when nothing but streaming happens.
constexpr int kManyMax = 160;
struct ManyArgs {
  const u32x4* src[kManyMax];
  int32_t first_piece[kManyMax + 1];  // prefix sums of the buffers' piece counts
  int n;
};
__global__ __launch_bounds__(512) void stream_read_many_kernel(ManyArgs a, uint32_t* __restrict__ sink) {
  constexpr int U = 8;
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 6), nw = (int64_t)gridDim.x * 8;
  const int64_t pieces = a.first_piece[a.n];
  uint32_t acc = 0;
  int b = 0;
  // Piece q of the sequence belongs to wave q % nw: at any moment the grid reads one contiguous window.  A wave
  // keeps U requests in flight all the time: the oldest is folded and its slot asked for the next piece at once
  // (a loop that issues U and then waits for all of them has nothing in flight half of the time).
  // the buffer of the current piece is kept in registers and looked up again only when q leaves it (q grows
  // monotonically and is wave-uniform): the table is a kernel argument indexed at run time, not something to
  // touch per request
  int64_t cur_first = 0, cur_end = a.first_piece[1];
  const u32x4* cur = a.src[0];
  auto request = [&](int64_t q) {
    u32x4 v = u32x4{0u, 0u, 0u, 0u};
    if (q < pieces) {
      while (q >= cur_end) {
        ++b;
        cur_first = a.first_piece[b], cur_end = a.first_piece[b + 1], cur = a.src[b];
      }
      v = __builtin_nontemporal_load(&cur[(q - cur_first) * 64 + lane]);
    }
    return v;
  };
  u32x4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) v[u] = request(wave + u * nw);
  for (int64_t p = wave; p < pieces; p += nw * U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
      v[u] = request(p + (U + u) * nw);
    }
  }
  if (acc == 0x9e3779b9u) sink[threadIdx.x] = acc;
}

// 8 waves per workgroup, 16 independent 16x16 accumulators per wave, operands drawn once from a generator
// (random mantissas and signs, exponents near 1: constant operands run faster than a real product does).
// v_mfma_f32_16x16x32_bf16 is the instruction the prefill GEMM uses; on random operands it sustains more than
// the 32x32x16 form does (the part is power-bound and this shape moves fewer accumulator registers per flop).
__global__ __launch_bounds__(512) void mfma_bf16_kernel(float* __restrict__ sink, int iters, uint32_t seed) {
  f32x4 acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  uint32_t r = seed + (blockIdx.x * 512 + threadIdx.x) * 2654435761u;
  auto draw = [&]() {
    u32x4 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      r = r * 1664525u + 1013904223u;
      v[j] = (r & 0x807f807fu) | 0x3f003f00u;  // +-[0.5, 1)
    }
    return __builtin_bit_cast(bf16x8, v);
  };
  bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = draw();
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = draw();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i & 3], b[i >> 2], acc[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += acc[i][0];
  if (s == 12345.678f) sink[threadIdx.x] = s;
}

// Every workgroup takes all of a CU's LDS and writes `pattern` over it (one workgroup per CU at a time; the grid is
// several times the CU count so that every CU gets one).
__global__ __launch_bounds__(256) void lds_fill_kernel(uint32_t pattern, uint32_t* __restrict__ sink, int words) {
  extern __shared__ __align__(16) uint32_t lds_all[];
  for (int i = threadIdx.x; i < words; i += 256) lds_all[i] = pattern;
  __syncthreads();
  if (lds_all[(threadIdx.x * 97) % words] != pattern) sink[threadIdx.x] = 1u;  // keeps the stores
}

}  // namespace

extern "C" int olmo355_probe_stream_read(const void* src, int64_t bytes, void* sink, void* stream) {
  if (!src || !sink || bytes < 1024) return O355_EINVAL;
  const int64_t pieces = bytes >> 10;
  // as in the small-M linears: enough waves that none holds more than a few pieces
  if (pieces >= 8 * 8 * 512) {
    const unsigned grid = (unsigned)std::min<int64_t>((pieces + 63) / 64, 4096);
    hipLaunchKernelGGL(stream_read_kernel<8>, dim3(grid), dim3(512), 0, as_stream(stream), (const u32x4*)src, pieces,
                       (uint32_t*)sink);
  } else {
    const unsigned grid = (unsigned)std::max<int64_t>((pieces + 15) / 16, 1);
    hipLaunchKernelGGL(stream_read_kernel<2>, dim3(grid), dim3(512), 0, as_stream(stream), (const u32x4*)src, pieces,
                       (uint32_t*)sink);
  }
  O355_CHECK_LAUNCH();
}

extern "C" int olmo355_probe_stream_read_many(const void* const* srcs, const int64_t* bytes, int n, void* sink,
                                              void* stream) {
  if (!srcs || !bytes || !sink || n < 1 || n > kManyMax) return O355_EINVAL;
  ManyArgs a;
  int64_t total = 0;
  for (int i = 0; i < n; ++i) {
    if (!srcs[i] || bytes[i] < 1024) return O355_EINVAL;
    a.src[i] = (const u32x4*)srcs[i];
    a.first_piece[i] = (int32_t)total;
    total += bytes[i] >> 10;
    if (total >= (1ll << 31)) return O355_EUNSUPPORTED;
  }
  a.first_piece[n] = (int32_t)total;
  a.n = n;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return O355_ELAUNCH;
  hipLaunchKernelGGL(stream_read_many_kernel, dim3((unsigned)(2 * cus)), dim3(512), 0, as_stream(stream), a, (uint32_t*)sink);
  O355_CHECK_LAUNCH();
}

// 256 workgroups x 8 waves x iters x 16 MFMAs of 16x16x32 (16384 flop each); *flops receives the total.
extern "C" int olmo355_probe_mfma_bf16(int iters, void* sink, double* flops, void* stream) {
  if (iters <= 0 || !sink) return O355_EINVAL;
  hipLaunchKernelGGL(mfma_bf16_kernel, dim3(256), dim3(512), 0, as_stream(stream), (float*)sink, iters, 77u);
  if (flops) *flops = 256.0 * 8.0 * (double)iters * 16.0 * 16384.0;
  O355_CHECK_LAUNCH();
}

// Leaves `pattern` in the LDS of every CU (tests run it before a kernel to show that the kernel reads nothing it has
// not written: LDS keeps what the last workgroup left there).
extern "C" int olmo355_probe_fill_lds(uint32_t pattern, void* sink, void* stream) {
  if (!sink) return O355_EINVAL;
  int dev = 0, cus = 0, lds = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess || cus <= 0 || lds < 65536)
    return O355_ELAUNCH;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(lds_fill_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
    return O355_ELAUNCH;
  hipLaunchKernelGGL(lds_fill_kernel, dim3((unsigned)(8 * cus)), dim3(256), (size_t)lds, as_stream(stream), pattern, (uint32_t*)sink, lds / 4);
  O355_CHECK_LAUNCH();
}
