// The gfx950 instructions that the MFMA stage-1 kernel names itself: matrix products, packed
// dot products, the half-wave swap, LDS operand reads, the direct global->LDS tile load, device-scope
// 128-bit accesses, scalar loads and the explicit wait counters. Everything else in the kernel is plain
// C++ over these, so this file is the whole of its dependence on the instruction set.
#ifndef FTA_GFX950_OPS_H
#define FTA_GFX950_OPS_H
#include "fta_device.h"

namespace fta {
namespace {

template <typename T> struct Mfma;
template <> struct Mfma<__bf16> {
  using Vec8 = bf16x8;
  using Vec4 = bf16x4;
  using Vec2 = bf16x2;
  static __device__ __forceinline__ f32x16 mma(Vec8 a, Vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // acc + v[0] + v[1]: one instruction sums a packed pair (and sums the ROUNDED values,
  // the very weights the P.V product applies)
  static __device__ __forceinline__ float add_pair(Vec2 v, float acc) {
    const Vec2 ones = {static_cast<__bf16>(1.f), static_cast<__bf16>(1.f)};
    return __builtin_amdgcn_fdot2_f32_bf16(v, ones, acc, false);
  }
};
template <> struct Mfma<_Float16> {
  using Vec8 = f16x8;
  using Vec4 = f16x4;
  using Vec2 = f16x2;
  static __device__ __forceinline__ f32x16 mma(Vec8 a, Vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float add_pair(Vec2 v, float acc) {
    const Vec2 ones = {static_cast<_Float16>(1.f), static_cast<_Float16>(1.f)};
    return __builtin_amdgcn_fdot2(v, ones, acc, false);
  }
};

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

#define FTA_GLOBAL __attribute__((address_space(1)))

// Lanes i and i+32 hold the same query row. v_permlane32_swap exchanges the upper half
// of its first operand with the lower half of its second; the partner's value is then
// in result 1 for lanes < 32 and in result 0 for lanes >= 32 (also when the compiler
// assigns both operands the same register, where both results hold the partner).
__device__ __forceinline__ float half_partner(float x, int lh) {
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, x), __builtin_bit_cast(unsigned, x), false, false);
  return __builtin_bit_cast(float, lh ? r[0] : r[1]);
}
__device__ __forceinline__ float half_swap_max(float x, int lh) { return fmaxf(x, half_partner(x, lh)); }
__device__ __forceinline__ float half_swap_sum(float x, int lh) { return x + half_partner(x, lh); }

// s_waitcnt vmcnt(N) only (expcnt / lgkmcnt left at "no wait"), gfx9 encoding.
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// Operand fragments are read from LDS with explicit instructions and explicit
// lgkmcnt waits. The compiler's own wait insertion treats every LDS read as possibly
// aliasing the in-flight global_load_lds writes of LATER tiles and would drain them
// (vmcnt 0) before each tile's reads, which defeats the multi-stage ring; reads it
// cannot see are not subject to that. LDS returns data in issue order, so
// "lgkmcnt <= N" means all but the N youngest reads have landed. The waited-for
// registers are threaded through the wait so that their consumers cannot move above it.
template <int OFF>
__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr) {
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
template <int OFF>
__device__ __forceinline__ u32x2 lds_read_tr16_b64(uint32_t addr) {
  u32x2 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
// Device-scope (sc1) 128-bit store / load: the store writes through to the point where
// every XCD sees it, the load is never served from a stale line of this XCD's caches.
// They carry the partials that one workgroup hands to another inside a launch without
// any cache-wide writeback or invalidate. Untracked like the reads above: wait_vmcnt.
__device__ __forceinline__ void store_b128_device(void* ptr, f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(ptr), "v"(v) : "memory");
}
__device__ __forceinline__ f32x4 load_b128_device(const void* ptr) {
  f32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=&v"(v) : "v"(ptr) : "memory");
  return v;
}
__device__ __forceinline__ void settle(f32x4& a) { asm volatile("" : "+v"(a)); }
// Scalar (wave-uniform) 32-bit loads of N block-table entries, requested together and
// waited for inside the same statement: the compiler would use vector loads (whose wait
// drains the tile requests in flight behind them), and a scalar register still in
// flight must not be visible to it, since it may move registers at will.
__device__ __forceinline__ void scalar_load_one(const int32_t* p0, int& a0) {
  asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=&s"(a0) : "s"(p0) : "memory");
}
__device__ __forceinline__ void scalar_load_pair(const int32_t* p0, const int32_t* p1, int& a0, int& a1) {
  asm volatile("s_load_dword %0, %2, 0x0\n\ts_load_dword %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
               : "=&s"(a0), "=&s"(a1) : "s"(p0), "s"(p1) : "memory");
}
__device__ __forceinline__ void scalar_load_quad(const int32_t* p0, const int32_t* p1, const int32_t* p2, const int32_t* p3,
                                                 int& a0, int& a1, int& a2, int& a3) {
  asm volatile("s_load_dword %0, %4, 0x0\n\ts_load_dword %1, %5, 0x0\n\ts_load_dword %2, %6, 0x0\n\t"
               "s_load_dword %3, %7, 0x0\n\ts_waitcnt lgkmcnt(0)"
               : "=&s"(a0), "=&s"(a1), "=&s"(a2), "=&s"(a3) : "s"(p0), "s"(p1), "s"(p2), "s"(p3) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_lgkm(u32x4& a) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(a) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_lgkm(u32x2& a, u32x2& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}

// A wave-uniform pointer, pinned to scalar registers: address arithmetic on it stays on the
// scalar unit and loads can use the (scalar base + 32-bit lane offset) addressing form.
__device__ __forceinline__ const char* uniform_ptr(const char* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
  return reinterpret_cast<const char*>((static_cast<uint64_t>(hi) << 32) | lo);
}

// Byte address of a dynamic-LDS pointer in the LDS address space (what ds_read takes).
__device__ __forceinline__ uint32_t lds_address(char* p) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((FTA_LDS char*)p));
}
// One wave-wide 16-byte-per-lane load from global memory straight into LDS: lane i's bytes land at
// lds_block + 16 * i (lds_block is wave-uniform). Counted by vmcnt like any vector load. A macro, not a
// function: the destination has to reach the builtin as an LDS-address-space pointer without a detour
// through a generic one.
#define FTA_LOAD_BLOCK_TO_LDS(lane_src, lds_block) \
  __builtin_amdgcn_global_load_lds((const FTA_GLOBAL void*)(lane_src), (FTA_LDS void*)(lds_block), 16, 0, 0)
// Occupancy the kernel is compiled for: exactly n waves per SIMD (which also fixes its register budget).
#define FTA_WAVES_PER_EU(n) __attribute__((amdgpu_waves_per_eu(n, n)))
// The workgroup barrier without the memory waits that __syncthreads adds (the kernel counts its own).
__device__ __forceinline__ void workgroup_barrier() { __builtin_amdgcn_s_barrier(); }
// Keeps the compiler from moving instructions across this point when it schedules.
__device__ __forceinline__ void schedule_fence() { __builtin_amdgcn_sched_barrier(0); }
// True in every lane if `pred` holds in any lane of the wave.
__device__ __forceinline__ bool wave_any(bool pred) { return __builtin_amdgcn_ballot_w64(pred) != 0; }

}  // namespace
}  // namespace fta
#endif  // FTA_GFX950_OPS_H
