// Host stand-in for the few HIP names that fta_device.h uses, so that its device functions (the
// dispatch order, the chunk choice, the block-wide reductions) can run on the CPU exactly as written:
// one host thread per GPU thread, std::barrier for __syncthreads, an exchange array per wave for
// __shfl_xor. Test infrastructure only; one block runs at a time (so `__shared__` is a plain static).
#pragma once
#include <algorithm>
#include <barrier>
#include <cmath>
#include <cstdint>
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
inline hipError_t hipLaunchKernel(const void*, dim3, dim3, void**, unsigned, hipStream_t) { return hipErrorUnknown; }

namespace host_block {
struct Block {
  unsigned threads;
  std::barrier<> all;
  std::vector<std::unique_ptr<std::barrier<>>> wave;
  std::vector<uint32_t> slot;
  explicit Block(unsigned n) : threads(n), all(n), slot(n) {
    for (unsigned w = 0; w < (n + 63) / 64; ++w) wave.emplace_back(new std::barrier<>(std::min(64u, n - 64 * w)));
  }
};
inline Block*& current() { static Block* b = nullptr; return b; }
}  // namespace host_block

inline thread_local dim3 threadIdx, blockIdx;
inline dim3 blockDim, gridDim;

inline void __syncthreads() { host_block::current()->all.arrive_and_wait(); }

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
  if (first != v) throw std::logic_error("readfirstlane on a value that differs between lanes");
  return first;
}
#define __builtin_amdgcn_readfirstlane(x) host_readfirstlane(x)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_logf(x) log2f(x)
using std::max;
using std::min;
