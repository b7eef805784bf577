// Host stand-in for the HIP names that the simpler kernels of this library use, so that their source
// runs on the CPU exactly as written: one host thread per GPU thread, std::barrier for __syncthreads,
// an exchange array per wave for __shfl_xor / ballot / readlane, a plain buffer for the dynamic LDS, and hipLaunchKernel
// = "run the grid, one workgroup after the other". TEST INFRASTRUCTURE ONLY: nothing under
// flash_tree_attn_amd/ includes or loads this; it exists so that device code can be checked against the
// oracle where no GPU is at hand (tests/test_dispatch_host.py, tests/test_host_block_kernels.py). Kernels
// that use matrix instructions or inline assembly cannot run here. One workgroup runs at a time, so
// `__shared__` is a plain static.
#pragma once
#include <algorithm>
#include <barrier>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <thread>
#include <vector>

#define __device__
#define __global__
#define __host__
#define __forceinline__ inline
#define __shared__ static
#define __launch_bounds__(...)

struct dim3 {
  unsigned x = 1, y = 1, z = 1;
  dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
typedef void* hipStream_t;
enum hipError_t { hipSuccess = 0, hipErrorUnknown = 1 };
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount };
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize };
inline hipError_t hipGetDevice(int* dev) { *dev = 0; return hipSuccess; }
inline hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t, int) { *value = 256; return hipSuccess; }
inline hipError_t hipFuncSetAttribute(const void*, hipFuncAttribute, int) { return hipSuccess; }

namespace host_block {
constexpr size_t kLdsBytes = 160 * 1024;
struct Block {
  unsigned threads;
  std::barrier<> all;
  std::vector<std::unique_ptr<std::barrier<>>> wave;
  std::vector<uint32_t> slot, slot2;
  explicit Block(unsigned n) : threads(n), all(n), slot(n), slot2(n) {
    for (unsigned w = 0; w < (n + 63) / 64; ++w) wave.emplace_back(new std::barrier<>(std::min(64u, n - 64 * w)));
  }
};
inline Block*& current() { static Block* b = nullptr; return b; }
inline char* dynamic_lds() { alignas(16) static char lds[kLdsBytes]; return lds; }
inline size_t& lds_limit() { static size_t bytes = 0; return bytes; }   // dynamic LDS the running launch asked for
}  // namespace host_block
#define FTA_DYNAMIC_LDS(name) char* name = host_block::dynamic_lds()

inline thread_local dim3 threadIdx, blockIdx;
inline dim3 blockDim, gridDim;

namespace host_block {
// Hook of a stand-in that keeps per-thread state of its own (gfx950_ops_host.h: loads in flight): called by every
// thread when it leaves the kernel.
struct Hooks {
  void (*at_thread_exit)() = nullptr;
};
inline Hooks& hooks() { static Hooks h; return h; }
}  // namespace host_block
inline void __syncthreads() { host_block::current()->all.arrive_and_wait(); }
inline void host_wave_barrier() { host_block::current()->wave[threadIdx.x / 64]->arrive_and_wait(); }

template <typename T>
inline T __shfl_xor(T v, int mask, int /*width*/) {
  static_assert(sizeof(T) == 4, "32-bit values");
  host_block::Block& b = *host_block::current();
  const unsigned t = threadIdx.x, w = t / 64;
  std::memcpy(&b.slot[t], &v, 4);
  b.wave[w]->arrive_and_wait();
  const unsigned src = (t & ~63u) | ((t ^ static_cast<unsigned>(mask)) & 63u);
  T r;
  std::memcpy(&r, &b.slot[src], 4);
  b.wave[w]->arrive_and_wait();
  return r;
}
// Value of the wave's first lane. The kernels only apply it to values that are the same in every lane,
// and the stand-in holds them to that.
inline int host_readfirstlane(int v) {
  const int first = __shfl_xor(v, static_cast<int>(threadIdx.x & 63), 64);   // lane ^ lane = lane 0
  if (first != v) {
    std::fprintf(stderr, "readfirstlane on a value that differs between lanes\n");
    std::abort();
  }
  return first;
}
#define __builtin_amdgcn_readfirstlane(x) host_readfirstlane(x)
// One bit per lane of the wave that holds `pred` (lanes the block does not have read as 0).
inline uint64_t host_ballot(bool pred) {
  host_block::Block& b = *host_block::current();
  const unsigned t = threadIdx.x, w = t / 64;
  b.slot[t] = pred ? 1u : 0u;
  b.wave[w]->arrive_and_wait();
  uint64_t bits = 0;
  for (unsigned l = 0; l < 64 && 64 * w + l < b.threads; ++l) bits |= static_cast<uint64_t>(b.slot[64 * w + l]) << l;
  b.wave[w]->arrive_and_wait();
  return bits;
}
#define __builtin_amdgcn_ballot_w64(pred) host_ballot(pred)
// Value of lane `sel` of the wave. The instruction takes the lane from a scalar register: the stand-in holds
// the callers to a selector that is the same in every lane.
inline int host_readlane(int v, int sel) {
  host_block::Block& b = *host_block::current();
  const unsigned t = threadIdx.x, w = t / 64;
  std::memcpy(&b.slot[t], &v, 4);
  b.slot2[t] = static_cast<uint32_t>(sel);
  b.wave[w]->arrive_and_wait();
  if (sel < 0 || sel > 63 || b.slot2[64 * w] != static_cast<uint32_t>(sel)) {
    std::fprintf(stderr, "readlane with a lane selector that differs between lanes\n");
    std::abort();
  }
  int r;
  std::memcpy(&r, &b.slot[64 * w + static_cast<unsigned>(sel)], 4);
  b.wave[w]->arrive_and_wait();
  return r;
}
#define __builtin_amdgcn_readlane(v, sel) host_readlane(v, sel)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_logf(x) log2f(x)
#define __builtin_amdgcn_fence(order, scope) ((void)0)
#define __builtin_amdgcn_wave_barrier() host_wave_barrier()
using std::max;
using std::min;

namespace host_block {
// Runs kern(params) for every workgroup of the grid in turn. A thread that returns from the kernel leaves the
// barriers (as a finished wave does on the GPU), so kernels whose threads exit at different points still end.
template <typename Kernel, typename Params>
inline hipError_t launch(Kernel kern, dim3 grid, dim3 block, const Params& params, size_t lds_bytes) {
  if (lds_bytes > kLdsBytes || block.x == 0 || block.x > 1024) return hipErrorUnknown;
  blockDim = block;
  gridDim = grid;
  lds_limit() = lds_bytes;
  for (unsigned id = 0; id < grid.x; ++id) {
    Block state(block.x);
    current() = &state;
    std::memset(dynamic_lds(), 0xFF, kLdsBytes);          // NaN patterns: nothing may be read before it is written
    std::vector<std::thread> pool;
    pool.reserve(block.x);
    for (unsigned t = 0; t < block.x; ++t)
      pool.emplace_back([&, t] {
        threadIdx = dim3(t);
        blockIdx = dim3(id);
        kern(params);
        if (hooks().at_thread_exit) hooks().at_thread_exit();
        state.all.arrive_and_drop();
        state.wave[t / 64]->arrive_and_drop();
      });
    for (auto& th : pool) th.join();
  }
  current() = nullptr;
  return hipSuccess;
}
}  // namespace host_block
// `kern` and `Params` are the kernel pointer and the parameter type in the scope of the library's
// launch_checked(), the only caller: the type-erased first argument cannot be called from here.
#define hipLaunchKernel(fn, grid, block, args, lds_bytes, stream) host_block::launch(kern, grid, block, *static_cast<const Params*>((args)[0]), lds_bytes)
