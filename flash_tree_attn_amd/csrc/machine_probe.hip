// Machine characterisation probes for gfx950, used by `bench.py --machine-probe`.
//
// Not part of the product path: a separate shared library (libfta_probe.so) with small
// kernels that measure what bounds the stage-1 kernel on the box at hand:
//   * the rate of dense v_mfma_f32_32x32x16_bf16 with one and two waves per SIMD, and the
//     shader clock the card holds while doing so (s_memtime against the 100 MHz
//     s_memrealtime);
//   * whether matrix and vector work of one SIMD overlap: a wave of MFMAs next to a wave
//     of FMAs ("roles"), against two waves that each interleave both ("mixed");
//   * the streaming rate of the kernel's HBM -> LDS load pattern (global_load_lds, 1 KiB
//     blocks of 4 rows) and of a plain register read, with one workgroup per CU.
// Every probe reports elapsed milliseconds (HIP events around `reps` launches) and the
// shader clock observed inside the kernel.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
#define PROBE_LDS __attribute__((address_space(3)))
#define PROBE_GLOBAL __attribute__((address_space(1)))

constexpr int kWorkgroups = 256;
constexpr int kMfmaPerIter = 16;    // per wave and iteration
constexpr int kFmaPerIter = 128;    // per wave and iteration

enum Role { kMatrix = 1, kVector = 2 };

// roles[slot]: what the wave in issue slot `slot` of its SIMD does (slot = order of arrival on the SIMD).
// mixed != 0: every wave interleaves one MFMA with eight FMAs instead.
template <int NT>
__global__ void __launch_bounds__(NT) compute_probe(float* sink, long long* clocks, int iters, int role0, int role1, int mixed) {
  __shared__ int arrivals[4];
  if (threadIdx.x < 4) arrivals[threadIdx.x] = 0;
  __syncthreads();
  const int simd = __builtin_amdgcn_s_getreg(2308) & 3;   // HW_ID[5:4]
  int slot = 0;
  if ((threadIdx.x & 63) == 0) slot = atomicAdd(&arrivals[simd], 1);
  slot = __shfl(slot, 0, 64);
  const int role = slot == 0 ? role0 : role1;
  f32x16 acc[4];
  for (int i = 0; i < 4; ++i)
    for (int e = 0; e < 16; ++e) acc[i][e] = threadIdx.x * 0.001f;
  // four different pseudo-random operand pairs in rotation: constant operands would not toggle the
  // multiplier inputs and understate the power the matrix pipeline draws on real data
  bf16x8 a[4], b[4];
  for (int j = 0; j < 4; ++j)
    for (int e = 0; e < 8; ++e) {
      unsigned h = (threadIdx.x * 8u + e) * 2654435761u + j * 40503u;
      h ^= h >> 13; h *= 0x5bd1e995u; h ^= h >> 15;
      a[j][e] = static_cast<__bf16>(((h & 0xffff) / 32768.0f - 1.0f));
      b[j][e] = static_cast<__bf16>(((h >> 16) / 32768.0f - 1.0f) * 0.5f);
    }
  float v[16];
  for (int e = 0; e < 16; ++e) v[e] = threadIdx.x * 0.5f + e;
  const float c1 = sink[0], c2 = sink[1];
  const long long t0 = clock64(), w0 = wall_clock64();
  if (mixed) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int r = 0; r < kMfmaPerIter; ++r) {
        acc[r & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(r >> 2) & 3], b[(r >> 2) & 3], acc[r & 3], 0, 0, 0);
#pragma unroll
        for (int e = 0; e < kFmaPerIter / kMfmaPerIter; ++e) v[(r & 1) * 8 + e] = __builtin_fmaf(v[(r & 1) * 8 + e], c1, c2);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  } else {
    for (int it = 0; it < iters; ++it) {
      if (role & kMatrix) {
#pragma unroll
        for (int r = 0; r < kMfmaPerIter; ++r) acc[r & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(r >> 2) & 3], b[(r >> 2) & 3], acc[r & 3], 0, 0, 0);
      }
      if (role & kVector) {
#pragma unroll
        for (int r = 0; r < kFmaPerIter / 16; ++r)
#pragma unroll
          for (int e = 0; e < 16; ++e) v[e] = __builtin_fmaf(v[e], c1, c2);
      }
    }
  }
  const long long t1 = clock64(), w1 = wall_clock64();
  float s = 0.f;
  for (int i = 0; i < 4; ++i)
    for (int e = 0; e < 16; ++e) s += acc[i][e];
  for (int e = 0; e < 16; ++e) s += v[e];
  if (s == 123.456f) sink[2] = s;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    clocks[0] = t1 - t0;
    clocks[1] = w1 - w0;
  }
}

// One workgroup of 512 threads streams `tiles` pairs of 16 KiB tiles (64 rows x 256 B each, the K and
// V tile of one step) from its own contiguous slice of the two buffers.
// dma != 0: global_load_lds into a 4-stage LDS ring, lane i -> row i%4, chunk i/4 of a 1 KiB block
// (the product kernel's pattern); dma == 0: plain 128-bit register loads.
__global__ void __launch_bounds__(512) stream_probe(const char* kbuf, const char* vbuf, int tiles, long long slice_bytes,
                                                     unsigned* sink, long long* clocks, int dma) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const char* kb = kbuf + static_cast<long long>(blockIdx.x) * slice_bytes;
  const char* vb = vbuf + static_cast<long long>(blockIdx.x) * slice_bytes;
  const int row = lane & 3, chunk = lane >> 2;
  unsigned acc = 0;
  const long long t0 = clock64(), w0 = wall_clock64();
  for (int t = 0; t < tiles; ++t) {
    char* ks = smem + (t & 3) * 32768;
    char* vs = ks + 16384;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int blk = i * 8 + wave;   // 4-row block 0..15 of the tile
      const long long off = static_cast<long long>(t) * 16384 + (blk * 4 + row) * 256 + chunk * 16;
      if (dma) {
        __builtin_amdgcn_global_load_lds((const PROBE_GLOBAL void*)(kb + off), (PROBE_LDS void*)(ks + blk * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const PROBE_GLOBAL void*)(vb + off), (PROBE_LDS void*)(vs + blk * 1024), 16, 0, 0);
      } else {
        const uint4 x = *reinterpret_cast<const uint4*>(kb + off);
        const uint4 y = *reinterpret_cast<const uint4*>(vb + off);
        acc ^= x.x ^ x.w ^ y.y ^ y.z;
      }
    }
    if (dma && (t & 3) == 3) {   // every fourth tile: drain, touch the ring, go on
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      acc ^= *reinterpret_cast<unsigned*>(smem + tid * 4 + (t & 4) * 1000);
      __syncthreads();
    }
  }
  __builtin_amdgcn_s_waitcnt(0);
  const long long t1 = clock64(), w1 = wall_clock64();
  if (acc == 0x12345) sink[0] = acc;
  if (blockIdx.x == 0 && tid == 0) {
    clocks[0] = t1 - t0;
    clocks[1] = w1 - w0;
  }
}

struct Buffers {
  float* sink = nullptr;
  long long* clocks = nullptr;
  char* kbuf = nullptr;
  char* vbuf = nullptr;
};

}  // namespace

extern "C" {

// which: 0 MFMA in one wave per SIMD (its partner idles); 1 MFMA in both waves of a SIMD; 2 FMA in one wave
// per SIMD (its partner idles); 3 roles (slot 0
// MFMA, slot 1 FMA); 4 mixed (both waves interleave MFMA and FMA); 5 stream HBM -> LDS (global_load_lds);
// 6 stream HBM -> registers. out[0] = milliseconds per launch, out[1] = shader clock in MHz inside the
// kernel, out[2] = work per launch (MFMA FLOPs for 0/1/3/4, FMA lane-ops for 2, bytes for 5/6).
// Returns 0, or -1 on a HIP error / unknown probe.
int fta_machine_probe(int which, int reps, double* out) {
  if (which < 0 || which > 6 || reps <= 0 || !out) return -1;
  Buffers b;
  const int iters = 2000, tiles = 128;
  const long long slice = static_cast<long long>(tiles) * 16384;       // per workgroup and buffer
  const size_t stream_bytes = static_cast<size_t>(kWorkgroups) * slice;  // 512 MiB per buffer
  if (hipMalloc(&b.sink, 64) != hipSuccess || hipMalloc(&b.clocks, 64) != hipSuccess) return -1;
  const float init[4] = {1.0001f, 0.5f, 0.f, 0.f};
  if (hipMemcpy(b.sink, init, sizeof(init), hipMemcpyHostToDevice) != hipSuccess) return -1;
  if (which >= 5) {
    if (hipMalloc(&b.kbuf, stream_bytes) != hipSuccess || hipMalloc(&b.vbuf, stream_bytes) != hipSuccess) return -1;
    if (hipMemset(b.kbuf, 1, stream_bytes) != hipSuccess || hipMemset(b.vbuf, 2, stream_bytes) != hipSuccess) return -1;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(stream_probe), hipFuncAttributeMaxDynamicSharedMemorySize, 131072) != hipSuccess)
      return -1;
  }
  auto launch = [&]() {
    switch (which) {
      case 0: hipLaunchKernelGGL(compute_probe<512>, dim3(kWorkgroups), dim3(512), 0, 0, b.sink, b.clocks, iters, kMatrix, 0, 0); break;
      case 1: hipLaunchKernelGGL(compute_probe<512>, dim3(kWorkgroups), dim3(512), 0, 0, b.sink, b.clocks, iters, kMatrix, kMatrix, 0); break;
      case 2: hipLaunchKernelGGL(compute_probe<512>, dim3(kWorkgroups), dim3(512), 0, 0, b.sink, b.clocks, iters, kVector, 0, 0); break;
      case 3: hipLaunchKernelGGL(compute_probe<512>, dim3(kWorkgroups), dim3(512), 0, 0, b.sink, b.clocks, iters, kMatrix, kVector, 0); break;
      case 4: hipLaunchKernelGGL(compute_probe<512>, dim3(kWorkgroups), dim3(512), 0, 0, b.sink, b.clocks, iters, 0, 0, 1); break;
      case 5: hipLaunchKernelGGL(stream_probe, dim3(kWorkgroups), dim3(512), 131072, 0, b.kbuf, b.vbuf, tiles, slice,
                                 reinterpret_cast<unsigned*>(b.sink), b.clocks, 1); break;
      default: hipLaunchKernelGGL(stream_probe, dim3(kWorkgroups), dim3(512), 131072, 0, b.kbuf, b.vbuf, tiles, slice,
                                  reinterpret_cast<unsigned*>(b.sink), b.clocks, 0); break;
    }
  };
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -1;
  for (int i = 0; i < 3; ++i) launch();   // warm-up
  int rc = hipEventRecord(e0, 0) == hipSuccess ? 0 : -1;
  for (int i = 0; i < reps; ++i) launch();
  if (hipEventRecord(e1, 0) != hipSuccess) rc = -1;
  if (hipEventSynchronize(e1) != hipSuccess || hipGetLastError() != hipSuccess) rc = -1;
  float ms = 0.f;
  if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) rc = -1;
  long long clk[2] = {0, 1};
  if (hipMemcpy(clk, b.clocks, sizeof(clk), hipMemcpyDeviceToHost) != hipSuccess) rc = -1;
  out[0] = ms / reps;
  out[1] = clk[1] > 0 ? static_cast<double>(clk[0]) / (clk[1] / 100.0) : 0.0;   // wall clock ticks at 100 MHz
  const double waves = 8.0 * kWorkgroups;
  const double mfma_flops = 2.0 * 32 * 32 * 16;
  switch (which) {
    case 1: case 4: out[2] = waves * iters * kMfmaPerIter * mfma_flops; break;
    case 0: case 3: out[2] = 0.5 * waves * iters * kMfmaPerIter * mfma_flops; break;
    case 2: out[2] = 0.5 * waves * iters * kFmaPerIter * 64.0; break;
    default: out[2] = 2.0 * stream_bytes; break;
  }
  // teardown: a failure here cannot be acted on, the measurement above stands or falls by rc
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(b.sink);
  (void)hipFree(b.clocks);
  if (b.kbuf) (void)hipFree(b.kbuf);
  if (b.vbuf) (void)hipFree(b.vbuf);
  return rc;
}

}  // extern "C"
