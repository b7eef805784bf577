// Host stand-ins for flash_tree_attn_amd/csrc/gfx950_ops.h, so that the MFMA stage-1 kernel's SOURCE
// runs on host threads exactly as written (see hip/hip_runtime.h for the execution model). TEST
// INFRASTRUCTURE ONLY. Include after fta_device.h and before the kernel: it claims the include guards
// of gfx950_ops.h and wide_loop_asm.inc, whose bodies (instructions, inline assembly) then drop out.
//
// What is modelled: the data movement and arithmetic of each instruction - the 32x32x16 matrix
// product with its operand and accumulator lane layout, the packed dot product, the half-wave swap,
// the plain and the transposing LDS reads (addresses are offsets into the workgroup's LDS buffer), the
// direct global->LDS load, ballots and barriers. Matrix products accumulate in fp32 in ascending k; the
// hardware's internal order may differ in the last bits.
//
// Time is modelled at its two extremes for the direct global->LDS loads, the only loads the kernel
// waits for by count. By default a load lands the moment it is issued, the earliest it ever could:
// a stage that is requested while another wave may still read it is then a data race for the thread
// sanitizer. With FTA_HOST_LOADS_LAND_LATE set in the environment a load lands only when a vmcnt wait
// of its wave forces it to (s_waitcnt vmcnt(N): all but the N youngest have landed; nothing else
// counts, not even __syncthreads, whose own wait the kernel does not rely on), the latest the hardware allows: a wait that allows one load too many, or a missing
// one, leaves NaN patterns in LDS for the products to find, reading a stage before the loading wave
// has waited and passed a barrier is a data race, and a load still in flight when its thread leaves
// the kernel aborts the run. (host_block_loads_land_late(int), exported by stage1_mfma_host.cpp, switches
// the mode between launches.) LDS operand reads are in flight until their lgkmcnt wait in both modes (see
// wait_lgkm below).
//
// The hand-scheduled 64-row-wave loop (wide_loop_asm.inc) is assembly over fixed registers: its macros
// abort here, unless the build supplies them as calls of the interpreter in gfx950_asm_host.h.
#pragma once
#define FTA_GFX950_OPS_H
#define FTA_WIDE_LOOP_ASM_INC
#include <deque>
#include <type_traits>

#include "fta_device.h"

namespace host_block {
[[noreturn]] inline void no_assembly() {
  std::fprintf(stderr, "the assembly loop of the 64-row-wave kernel cannot run on the host\n");
  std::abort();
}
// One exchange area per wave for the cross-lane instructions: 64 lanes x 64 bytes.
struct WaveExchange {
  alignas(16) unsigned char bytes[64][64];
};
inline WaveExchange* exchange() { static WaveExchange x[16]; return x; }
inline unsigned lane_id() { return threadIdx.x & 63; }
inline WaveExchange& my_exchange() { return exchange()[threadIdx.x / 64]; }
// Address of LDS byte `addr`, bounds-checked for an access of `bytes` bytes against what the launch asked for.
// A direct global->LDS load of this lane that has not landed yet (late-landing mode).
struct LoadInFlight {
  const char* src;        // null: a load into registers (load_b128_device), its 16 bytes in `data`
  uint32_t lds_addr;
  unsigned char data[16] = {};
};
inline bool& loads_land_late() { static bool late = std::getenv("FTA_HOST_LOADS_LAND_LATE") != nullptr; return late; }   // also host_block_loads_land_late()
inline std::deque<LoadInFlight>& loads_in_flight() { static thread_local std::deque<LoadInFlight> q; return q; }
inline char* lds_at(uint32_t addr, uint32_t bytes);
// Lands the oldest loads of this lane until at most `allowed` are in flight (the counter retires in issue order).
// Loads into registers that a wait has landed and no settle() has handed to its register yet, oldest first.
inline std::deque<LoadInFlight>& landed_register_loads() { static thread_local std::deque<LoadInFlight> q; return q; }
inline void land_all_but(size_t allowed) {
  std::deque<LoadInFlight>& q = loads_in_flight();
  while (q.size() > allowed) {
    if (q.front().src) std::memcpy(lds_at(q.front().lds_addr, 16), q.front().src, 16);
    else landed_register_loads().push_back(q.front());
    q.pop_front();
  }
}
// An LDS operand read of this lane whose data no lgkmcnt wait has handed to a register yet.
struct LdsReadInFlight {
  unsigned char data[16];
};
inline std::deque<LdsReadInFlight>& lds_reads_in_flight() { static thread_local std::deque<LdsReadInFlight> q; return q; }
inline void no_load_may_outlive_its_thread() {
  if (!loads_in_flight().empty()) {
    std::fprintf(stderr, "a thread left the kernel with %zu global->LDS loads in flight\n", loads_in_flight().size());
    std::abort();
  }
  if (!landed_register_loads().empty()) {
    std::fprintf(stderr, "a thread left the kernel with %zu loaded registers that no settle() took\n", landed_register_loads().size());
    std::abort();
  }
  if (!lds_reads_in_flight().empty()) {
    std::fprintf(stderr, "a thread left the kernel with %zu LDS operand reads that no wait has landed\n", lds_reads_in_flight().size());
    std::abort();
  }
}
inline const bool hooks_installed = [] {
  hooks().at_thread_exit = no_load_may_outlive_its_thread;
  return true;
}();
inline char* lds_at(uint32_t addr, uint32_t bytes) {
  if (static_cast<size_t>(addr) + bytes > lds_limit()) {
    std::fprintf(stderr, "LDS access of %u bytes at %u beyond the %zu bytes of this launch\n", bytes, addr, lds_limit());
    std::abort();
  }
  return dynamic_lds() + addr;
}
}  // namespace host_block

#define FTA_WAVES_PER_EU(n)
#define __HIP_MEMORY_SCOPE_AGENT 4
// The assembly statements of the 64-row-wave loop: absent (a kernel that reaches one aborts), unless the build
// names a rendering of them as interpreter calls (FTA_HOST_WIDE_LOOP_INC, made from the same generator output as
// wide_loop_asm.inc by tests/test_host_block_wide.py; included at the end of this file).
#ifndef FTA_HOST_WIDE_LOOP_INC
#define FTA_WIDE_LOOP_128_BF16() host_block::no_assembly()
#define FTA_WIDE_LOOP_128_F16() host_block::no_assembly()
#define FTA_WIDE_LOOP_64_BF16() host_block::no_assembly()
#define FTA_WIDE_LOOP_64_F16() host_block::no_assembly()
#define FTA_WIDE_MASKED_128_BF16_H0() host_block::no_assembly()
#define FTA_WIDE_MASKED_128_BF16_H1() host_block::no_assembly()
#define FTA_WIDE_MASKED_128_F16_H0() host_block::no_assembly()
#define FTA_WIDE_MASKED_128_F16_H1() host_block::no_assembly()
#define FTA_WIDE_MASKED_64_BF16_H0() host_block::no_assembly()
#define FTA_WIDE_MASKED_64_BF16_H1() host_block::no_assembly()
#define FTA_WIDE_MASKED_64_F16_H0() host_block::no_assembly()
#define FTA_WIDE_MASKED_64_F16_H1() host_block::no_assembly()
#endif

namespace fta {
namespace {

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

// v_mfma_f32_32x32x16: D[m][n] = C[m][n] + sum_k A[m][k] B[n][k], k = 0..15. Lane (i = lane % 32,
// h = lane / 32) supplies A[i][8h .. 8h+7] and B[i][8h .. 8h+7]; it holds D[m][i] for
// m = 8 (r / 4) + 4 h + r % 4, r = 0..15.
template <typename Vec8>
inline f32x16 host_mfma_32x32x16(Vec8 a, Vec8 b, f32x16 c) {
  host_block::WaveExchange& x = host_block::my_exchange();
  const unsigned lane = host_block::lane_id(), i = lane & 31, h = lane >> 5;
  float* mine = reinterpret_cast<float*>(x.bytes[lane]);
  for (int e = 0; e < 8; ++e) {
    mine[e] = static_cast<float>(a[e]);
    mine[8 + e] = static_cast<float>(b[e]);
  }
  host_wave_barrier();
  f32x16 d = c;
  for (int r = 0; r < 16; ++r) {
    const unsigned m = 8 * (r / 4) + 4 * h + r % 4;
    float acc = c[r];
    for (unsigned k = 0; k < 16; ++k) {
      const float* arow = reinterpret_cast<const float*>(x.bytes[m + 32 * (k / 8)]);        // lane that holds A[m][k]
      const float* bcol = reinterpret_cast<const float*>(x.bytes[i + 32 * (k / 8)]) + 8;    // lane that holds B[i][k]
      acc += arow[k % 8] * bcol[k % 8];
    }
    d[r] = acc;
  }
  host_wave_barrier();
  return d;
}

template <typename T> struct Mfma;
template <> struct Mfma<__bf16> {
  using Vec8 = bf16x8;
  using Vec4 = bf16x4;
  using Vec2 = bf16x2;
  static inline f32x16 mma(Vec8 a, Vec8 b, f32x16 c) { return host_mfma_32x32x16(a, b, c); }
  static inline float add_pair(Vec2 v, float acc) { return acc + static_cast<float>(v[0]) + static_cast<float>(v[1]); }
};
template <> struct Mfma<_Float16> {
  using Vec8 = f16x8;
  using Vec4 = f16x4;
  using Vec2 = f16x2;
  static inline f32x16 mma(Vec8 a, Vec8 b, f32x16 c) { return host_mfma_32x32x16(a, b, c); }
  static inline float add_pair(Vec2 v, float acc) { return acc + static_cast<float>(v[0]) + static_cast<float>(v[1]); }
};

// Value of the same register in the lane 32 away.
inline float half_partner(float x, int /*lh*/) { return __shfl_xor(x, 32, 64); }
inline float half_swap_max(float x, int lh) { return fmaxf(x, half_partner(x, lh)); }
inline float half_swap_sum(float x, int lh) { return x + half_partner(x, lh); }

template <int N> inline void wait_vmcnt() { host_block::land_all_but(N); }
// LDS operand reads are asynchronous too: the destination registers hold nothing until an
// s_waitcnt lgkmcnt(N) has let all but the N youngest reads land (LDS returns data in issue order).
// The kernel issues such reads ahead of their use and names, at each wait, the registers that the
// wait makes valid. Here a read returns a NaN pattern and queues its data; a wait hands the data of
// the reads it lands to the registers it names, and insists that these are exactly the reads it lands:
// a count that is one too high leaves the pattern in place (and aborts), one too low lands a read that
// no register is named for (and aborts).
namespace lds_reads {
inline std::deque<host_block::LdsReadInFlight>& queue() { return host_block::lds_reads_in_flight(); }
template <typename V> inline V issue(const void* data) {
  host_block::LdsReadInFlight r;
  std::memcpy(r.data, data, sizeof(V));
  queue().push_back(r);
  V poison;
  std::memset(&poison, 0xFF, sizeof(V));
  return poison;
}
template <typename V> inline void land_into(V& reg) {
  std::memcpy(&reg, queue().front().data, sizeof(V));
  queue().pop_front();
}
inline void expect_landing(size_t allowed_in_flight, size_t named) {
  if (queue().size() != allowed_in_flight + named) {
    std::fprintf(stderr, "s_waitcnt lgkmcnt(%zu) with %zu LDS reads in flight names %zu register group(s)\n", allowed_in_flight, queue().size(), named);
    std::abort();
  }
}
}  // namespace lds_reads
template <int N> inline void wait_lgkm(u32x4& a) {
  lds_reads::expect_landing(N, 1);
  lds_reads::land_into(a);
}
template <int N> inline void wait_lgkm(u32x2& a, u32x2& b) {
  lds_reads::expect_landing(N, 2);
  lds_reads::land_into(a);
  lds_reads::land_into(b);
}
// load_b128_device is a load the compiler does not see: the register holds nothing until a vmcnt wait has
// landed the load (modelled in both load modes; with global->LDS loads that land when issued the count only
// holds for vmcnt(0), the one wait the kernel uses for these), and settle() is where the kernel takes the value.
inline void settle(f32x4& a) {
  std::deque<host_block::LoadInFlight>& q = host_block::landed_register_loads();
  if (q.empty()) {
    std::fprintf(stderr, "settle() of a register whose load no vmcnt wait has landed\n");
    std::abort();
  }
  std::memcpy(&a, q.front().data, 16);
  q.pop_front();
}

template <int OFF>
inline u32x4 lds_read_b128(uint32_t addr) {
  return lds_reads::issue<u32x4>(host_block::lds_at(addr + OFF, 16));
}
// ds_read_b64_tr_b16: the 16 lanes of a group each fetch 8 bytes (four 16-bit values). The 64 values of
// the group, read as four rows of sixteen (row e = the values of lanes 4e .. 4e+3 in order), come back
// transposed: lane s receives element s of each row, i.e. value s % 4 of lane 4e + s / 4 for e = 0..3.
template <int OFF>
inline u32x2 lds_read_tr16_b64(uint32_t addr) {
  host_block::WaveExchange& x = host_block::my_exchange();
  const unsigned lane = host_block::lane_id(), s = lane & 15, group = lane & ~15u;
  std::memcpy(x.bytes[lane], host_block::lds_at(addr + OFF, 8), 8);
  host_wave_barrier();
  uint16_t out[4];
  for (unsigned e = 0; e < 4; ++e) {
    const unsigned src = group + 4 * e + s / 4;
    std::memcpy(&out[e], x.bytes[src] + 2 * (s % 4), 2);
  }
  host_wave_barrier();
  return lds_reads::issue<u32x2>(out);
}

inline void store_b128_device(void* ptr, f32x4 v) { std::memcpy(ptr, &v, 16); }
inline f32x4 load_b128_device(const void* ptr) {
  host_block::LoadInFlight load{nullptr, 0};
  std::memcpy(load.data, ptr, 16);
  host_block::loads_in_flight().push_back(load);
  f32x4 v;
  std::memset(&v, 0xFF, 16);
  return v;
}
inline void scalar_load_one(const int32_t* p0, int& a0) { a0 = *p0; }
inline void scalar_load_pair(const int32_t* p0, const int32_t* p1, int& a0, int& a1) { a0 = *p0; a1 = *p1; }
inline void scalar_load_quad(const int32_t* p0, const int32_t* p1, const int32_t* p2, const int32_t* p3, int& a0, int& a1, int& a2, int& a3) {
  a0 = *p0; a1 = *p1; a2 = *p2; a3 = *p3;
}
// The kernel promises a wave-uniform pointer: hold it to that.
inline const char* uniform_ptr(const char* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = static_cast<uint32_t>(host_readfirstlane(static_cast<int>(static_cast<uint32_t>(v))));
  const uint32_t hi = static_cast<uint32_t>(host_readfirstlane(static_cast<int>(static_cast<uint32_t>(v >> 32))));
  return reinterpret_cast<const char*>((static_cast<uint64_t>(hi) << 32) | lo);
}
inline uint32_t lds_address(char* p) { return static_cast<uint32_t>(p - host_block::dynamic_lds()); }
// global_load_lds, 16 bytes per lane: the destination block must be wave-uniform.
inline void host_load_block_to_lds(const char* lane_src, char* lds_block) {
  const uint32_t base = lds_address(lds_block);
  (void)uniform_ptr(lds_block);
  const uint32_t mine = base + 16 * host_block::lane_id();
  if (host_block::loads_land_late()) {
    (void)host_block::lds_at(mine, 16);                        // the bounds check, at issue
    host_block::loads_in_flight().push_back({lane_src, mine});
  } else {
    std::memcpy(host_block::lds_at(mine, 16), lane_src, 16);
  }
}
#define FTA_LOAD_BLOCK_TO_LDS(lane_src, lds_block) host_load_block_to_lds(lane_src, lds_block)
inline void workgroup_barrier() { host_block::current()->all.arrive_and_wait(); }   // s_barrier alone: no wait for memory operations
inline void schedule_fence() {}
inline bool wave_any(bool pred) {
  int any = pred ? 1 : 0;
  for (int m = 1; m < 64; m <<= 1) any |= __shfl_xor(any, m, 64);
  return any != 0;
}

}  // namespace
}  // namespace fta

#ifdef FTA_HOST_WIDE_LOOP_INC
#include "gfx950_asm_host.h"
#include FTA_HOST_WIDE_LOOP_INC
#endif
