// Runs the host build of the library (see hip/hip_runtime.h in this directory) under the address and
// undefined-behaviour sanitizers: every buffer is allocated at exactly its size, so a kernel that reads or
// writes one element past a tensor, a page or the scratch is reported. Also checks the results against a
// plain double-precision attention, so that the run is not vacuous. Exit code 0 = clean.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "fta.h"

extern "C" void host_block_loads_land_late(int late) __attribute__((weak));   // only in builds with the MFMA kernel

namespace {
struct Case {
  int bsz, hq, hkv, L, D, tmax, splits, page;   // page 0 = contiguous caches
  std::vector<long long> lens;
  bool packed;
  bool mfma = false;    // bf16 tensors through the MFMA kernel (where the build has it) instead of fp32 through the shuffle kernel
  bool fused = false;   // with counters: the merge inside stage 1's launch
  bool key_halves = false;   // the MFMA kernel's form for small units: two waves per 32-row block
  bool wide = false;         // the MFMA kernel's 64-row-wave form, its assembly statements interpreted
};

std::mt19937 rng(1234);
float rnd() { return std::normal_distribution<float>(0.f, 1.f)(rng); }
uint16_t to_bf16(float x) {
  uint32_t u;
  std::memcpy(&u, &x, 4);
  return static_cast<uint16_t>((u + 0x7FFF + ((u >> 16) & 1)) >> 16);
}
float from_bf16(uint16_t h) {
  const uint32_t u = static_cast<uint32_t>(h) << 16;
  float x;
  std::memcpy(&x, &u, 4);
  return x;
}
// Rounds `t` to bf16 in place (the reference then sees what the library sees) and returns the 16-bit tensor; NaN stays NaN.
std::vector<uint16_t> as_bf16(std::vector<float>& t) {
  std::vector<uint16_t> h(t.size());
  for (size_t i = 0; i < t.size(); ++i) {
    h[i] = std::isnan(t[i]) ? uint16_t{0x7FC0} : to_bf16(t[i]);
    t[i] = from_bf16(h[i]);
  }
  return h;
}

int run(const Case& c) {
  const int G = c.hq / c.hkv;
  std::vector<float> q((size_t)c.bsz * c.hq * c.L * c.D), ck((size_t)c.bsz * c.hkv * c.L * c.D), cv(ck.size());
  std::vector<float> k((size_t)c.bsz * c.hkv * c.tmax * c.D), v(k.size());
  for (auto* t : {&q, &ck, &cv, &k, &v}) for (auto& x : *t) x = rnd();
  // a random tree: row i attends to itself and its ancestors
  std::vector<int> parent(c.L, -1);
  for (int i = 1; i < c.L; ++i) parent[i] = rng() % i;
  std::vector<float> mask((size_t)c.L * c.L, -INFINITY);
  std::vector<unsigned long long> bits((size_t)c.L * ((c.L + 63) / 64), 0);
  for (int i = 0; i < c.L; ++i)
    for (int j = i; j >= 0; j = parent[j]) {
      mask[(size_t)i * c.L + j] = 0.f;
      bits[(size_t)i * ((c.L + 63) / 64) + j / 64] |= 1ull << (j % 64);
    }
  std::vector<float> out((size_t)c.bsz * c.hq * c.L * c.D, NAN);

  // paged form of the caches: pages in reversed order, table exactly as wide as needed
  std::vector<float> kp, vp;
  std::vector<int32_t> table;
  const int per_seq = c.page ? (c.tmax + c.page - 1) / c.page : 0;
  if (c.page) {
    const int pages = c.bsz * per_seq;
    kp.assign((size_t)pages * c.hkv * c.page * c.D, NAN);
    vp.assign(kp.size(), NAN);
    table.resize((size_t)c.bsz * per_seq);
    for (int b = 0; b < c.bsz; ++b)
      for (int pg = 0; pg < per_seq; ++pg) {
        const int phys = pages - 1 - (b * per_seq + pg);
        table[(size_t)b * per_seq + pg] = phys;
        for (int h = 0; h < c.hkv; ++h)
          for (int r = 0; r < c.page && pg * c.page + r < c.tmax; ++r) {
            const size_t src = (((size_t)b * c.hkv + h) * c.tmax + pg * c.page + r) * c.D;
            const size_t dst = (((size_t)phys * c.hkv + h) * c.page + r) * c.D;
            std::memcpy(&kp[dst], &k[src], sizeof(float) * c.D);
            std::memcpy(&vp[dst], &v[src], sizeof(float) * c.D);
          }
      }
  }

  std::vector<uint16_t> q16, ck16, cv16, k16, v16, kp16, vp16, out16;
  if (c.mfma) {
    q16 = as_bf16(q); ck16 = as_bf16(ck); cv16 = as_bf16(cv);
    if (c.page) { kp16 = as_bf16(kp); vp16 = as_bf16(vp); }
    k16 = as_bf16(k); v16 = as_bf16(v);       // rounded also when paged: the reference reads k and v
    if (c.page) { k16.clear(); v16.clear(); k16.shrink_to_fit(); v16.shrink_to_fit(); }
    out16.assign(out.size(), 0x7FC0);
  }
  fta_args a{};
  a.kv_seq_len = c.lens.data();
  if (c.mfma) {
    a.q = q16.data(); a.cur_k = ck16.data(); a.cur_v = cv16.data(); a.out = out16.data();
    a.k_cache = c.page ? kp16.data() : k16.data();
    a.v_cache = c.page ? vp16.data() : v16.data();
  } else {
    a.q = q.data(); a.cur_k = ck.data(); a.cur_v = cv.data(); a.out = out.data();
    a.k_cache = c.page ? kp.data() : k.data();
    a.v_cache = c.page ? vp.data() : v.data();
  }
  a.mask = c.packed ? (const void*)bits.data() : (const void*)mask.data();
  a.mask_kind = c.packed ? FTA_MASK_PACKED_U64 : FTA_MASK_ADDITIVE_F32;
  a.bsz = c.bsz; a.num_q_heads = c.hq; a.num_kv_heads = c.hkv; a.cur_heads = c.hkv; a.q_len = c.L; a.head_dim = c.D;
  a.block_size = 64; a.dtype = c.mfma ? FTA_BF16 : FTA_F32; a.len_dtype = FTA_I64; a.force_splits = c.splits;
  a.force_kernel = c.wide ? FTA_KERNEL_MFMA_WIDE : c.key_halves ? FTA_KERNEL_MFMA_SPLIT_KEYS : c.mfma ? FTA_KERNEL_MFMA : FTA_KERNEL_SHUFFLE;
  a.sm_scale = 1.f / std::sqrt((float)c.D);
  const long long LD = (long long)c.L * c.D;
  a.q_stride[0] = c.hq * LD; a.q_stride[1] = LD; a.q_stride[2] = c.D;
  a.ck_stride[0] = a.cv_stride[0] = c.hkv * LD; a.ck_stride[1] = a.cv_stride[1] = LD; a.ck_stride[2] = a.cv_stride[2] = c.D;
  a.out_stride[0] = c.hq * LD; a.out_stride[1] = LD; a.out_stride[2] = c.D;
  if (c.page) {
    a.block_table = table.data(); a.block_table_stride = per_seq; a.page_size = c.page;
    a.cache_len = a.v_cache_len = per_seq * c.page;
    a.k_stride[0] = a.v_stride[0] = (long long)c.hkv * c.page * c.D; a.k_stride[1] = a.v_stride[1] = (long long)c.page * c.D;
  } else {
    a.cache_len = a.v_cache_len = c.tmax;
    a.k_stride[0] = a.v_stride[0] = (long long)c.hkv * c.tmax * c.D; a.k_stride[1] = a.v_stride[1] = (long long)c.tmax * c.D;
  }
  a.k_stride[2] = a.v_stride[2] = c.D;
  a.mask_stride[0] = a.mask_stride[1] = 0; a.mask_stride[2] = c.packed ? (c.L + 63) / 64 : c.L;
  fta_plan_out pl{};
  if (int st = fta_plan(&a, 256, &pl)) { std::printf("plan failed %d\n", st); return 1; }
  std::vector<float> mid((size_t)pl.mid_o_elems), lse((size_t)pl.mid_lse_elems);
  if (pl.num_splits > 1) {
    a.mid_o = mid.data(); a.mid_lse = lse.data(); a.mid_splits = pl.num_splits;
    a.mid_o_stride[0] = (long long)c.hq * pl.num_splits * LD; a.mid_o_stride[1] = pl.num_splits * LD; a.mid_o_stride[2] = LD; a.mid_o_stride[3] = c.D;
    a.mid_lse_stride[0] = (long long)c.hq * pl.num_splits * c.L; a.mid_lse_stride[1] = (long long)pl.num_splits * c.L; a.mid_lse_stride[2] = c.L;
  }
  std::vector<int32_t> counters(c.fused ? (size_t)pl.counter_elems : 0, 0);
  if (c.fused) {
    if (pl.counter_elems <= 0) { std::printf("no merge inside the launch for this case\n"); return 1; }
    a.counters = counters.data(); a.counter_elems = pl.counter_elems;
  }
  if (int st = fta_decode(&a, nullptr)) { std::printf("decode failed %d\n", st); return 1; }
  for (int32_t n : counters) if (n != 0) { std::printf("a counter was left at %d\n", n); return 1; }
  if (c.mfma) for (size_t i = 0; i < out.size(); ++i) out[i] = from_bf16(out16[i]);

  // plain attention in double
  double worst = 0;
  for (int b = 0; b < c.bsz; ++b) {
    const int T = (int)std::min<long long>(std::max<long long>(c.lens[b], 0), a.cache_len);
    for (int h = 0; h < c.hq; ++h)
      for (int i = 0; i < c.L; ++i) {
        const float* qr = &q[(((size_t)b * c.hq + h) * c.L + i) * c.D];
        std::vector<double> s(T + c.L);
        double mx = -INFINITY;
        for (int j = 0; j < T + c.L; ++j) {
          const float* kr = j < T ? &k[(((size_t)b * c.hkv + h / G) * c.tmax + j) * c.D] : &ck[(((size_t)b * c.hkv + h / G) * c.L + (j - T)) * c.D];
          double d = 0;
          for (int e = 0; e < c.D; ++e) d += (double)qr[e] * kr[e];
          s[j] = d * a.sm_scale + (j < T ? 0.0 : (double)mask[(size_t)i * c.L + (j - T)]);
          mx = std::max(mx, s[j]);
        }
        double den = 0;
        std::vector<double> o(c.D, 0.0);
        for (int j = 0; j < T + c.L; ++j) {
          const double p = std::exp(s[j] - mx);
          den += p;
          const float* vr = j < T ? &v[(((size_t)b * c.hkv + h / G) * c.tmax + j) * c.D] : &cv[(((size_t)b * c.hkv + h / G) * c.L + (j - T)) * c.D];
          for (int e = 0; e < c.D; ++e) o[e] += p * vr[e];
        }
        for (int e = 0; e < c.D; ++e) {
          const double ref = o[e] / den, got = out[(((size_t)b * c.hq + h) * c.L + i) * c.D + e];
          const double err = std::fabs(ref - got);                      // NaN (an element never written) must fail
          worst = err == err ? std::max(worst, c.mfma ? err / (1.0 + 5.0 * std::fabs(ref)) : err) : INFINITY;
        }
      }
  }
  std::printf("%s bsz %d hq %d hkv %d L %d D %d tmax %d splits %d page %d packed %d: plan %d x %d, %d rows per workgroup, max abs err %.2e\n",
              c.mfma ? "bf16/mfma" : "fp32/shuffle", c.bsz, c.hq, c.hkv, c.L, c.D, c.tmax, c.splits, c.page, (int)c.packed, pl.num_splits, pl.chunk,
              pl.rows_per_wg, worst);
  return worst < (c.mfma ? 2e-3 : 2e-5) ? 0 : 1;   // bf16: 2e-3 absolute + 1e-2 relative, as everywhere
}
// The accepted-path append on exactly sized caches, one sequence running into the end of its cache.
int run_append() {
  const int bsz = 2, hkv = 2, L = 5, D = 32, tmax = 32, max_acc = 3;
  std::vector<float> k((size_t)bsz * hkv * tmax * D), v(k.size()), ck((size_t)bsz * hkv * L * D), cv(ck.size());
  for (auto* t : {&k, &v, &ck, &cv}) for (auto& x : *t) x = rnd();
  std::vector<float> k_ref = k, v_ref = v;
  std::vector<int32_t> idx = {0, 4, 2, 1, 3, 0};
  std::vector<long long> acc = {3, 2}, lens = {30, 7}, want = {32, 9};
  for (int b = 0; b < bsz; ++b)
    for (int a = 0; a < acc[b]; ++a)
      if (lens[b] + a < tmax)
        for (int h = 0; h < hkv; ++h) {
          std::memcpy(&k_ref[(((size_t)b * hkv + h) * tmax + lens[b] + a) * D], &ck[(((size_t)b * hkv + h) * L + idx[b * max_acc + a]) * D], sizeof(float) * D);
          std::memcpy(&v_ref[(((size_t)b * hkv + h) * tmax + lens[b] + a) * D], &cv[(((size_t)b * hkv + h) * L + idx[b * max_acc + a]) * D], sizeof(float) * D);
        }
  fta_append_args a{};
  a.k_cache = k.data(); a.v_cache = v.data(); a.cur_k = ck.data(); a.cur_v = cv.data();
  a.accept_idx = idx.data(); a.accept_len = acc.data(); a.kv_seq_len = lens.data(); a.kv_seq_len_out = lens.data();
  a.bsz = bsz; a.num_kv_heads = hkv; a.q_len = L; a.head_dim = D; a.cache_len = tmax; a.max_accept = max_acc;
  a.dtype = FTA_F32; a.len_dtype = FTA_I64; a.accept_idx_stride = max_acc;
  a.k_stride[0] = a.v_stride[0] = (long long)hkv * tmax * D; a.k_stride[1] = a.v_stride[1] = (long long)tmax * D; a.k_stride[2] = a.v_stride[2] = D;
  a.ck_stride[0] = a.cv_stride[0] = (long long)hkv * L * D; a.ck_stride[1] = a.cv_stride[1] = (long long)L * D; a.ck_stride[2] = a.cv_stride[2] = D;
  if (int st = fta_append_kv(&a, nullptr)) { std::printf("append failed %d\n", st); return 1; }
  const bool same = k == k_ref && v == v_ref && lens == want;
  std::printf("append: %s\n", same ? "bit-exact" : "DIFFERS");
  return same ? 0 : 1;
}
}  // namespace

int main(int argc, char** argv) {
  // "mfma" as first argument: the build holds the MFMA kernel (stage1_mfma_host.cpp), run its cases as well;
  // "both" as second: run them once with global->LDS loads that land when issued and once with loads that land
  // only when a wait forces them to (a stage read before its loader has waited and passed a barrier is then a race)
  const bool with_mfma = argc > 1 && std::strcmp(argv[1], "mfma") == 0;
  const bool both = with_mfma && argc > 2 && std::strcmp(argv[2], "both") == 0;
  const Case mfma_cases[] = {
      {2, 4, 2, 5, 64, 200, 2, 0, {200, 77}, false, true},                 // 4 waves, rings of 2; ragged last tiles
      {1, 8, 1, 20, 128, 390, 1, 0, {390}, false, true},                   // 8 waves pipelined through rings of 3 and 5, ragged end
      {2, 2, 2, 3, 128, 160, 2, 16, {160, 17}, true, true},                // paged, packed mask
      {2, 8, 1, 20, 64, 192, 3, 0, {192, 70}, false, true, true},          // pipelined, merge inside the launch
      {1, 2, 2, 3, 256, 65, 1, 0, {65}, false, true},                      // head_dim 256, one key past a tile
      {2, 2, 2, 26, 128, 161, 2, 0, {161, 33}, false, true, false, true},  // key halves: 26 rows, one key in the upper half of a tile
      {2, 4, 1, 16, 64, 160, 2, 16, {160, 70}, true, true, true, true},    // key halves: 64 rows, paged, packed mask, merge inside the launch
      {1, 4, 1, 64, 128, 300, 1, 0, {300}, false, true, false, false, true},           // 64-row waves: tree tile, 4 tiles in the loop, ragged tail
      {2, 8, 1, 32, 64, 200, 2, 0, {200, 64}, true, true, true, false, true},          // 64-row waves: head_dim 64, packed mask, merge inside the launch
  };
  const Case cases[] = {
      {2, 4, 2, 5, 32, 100, 2, 0, {100, 37}, false},          // ragged tiles at the end of cache and tree
      {2, 2, 1, 3, 64, 129, 3, 0, {129, 0}, true},            // one key past a tile boundary; an empty cache; packed mask
      {1, 2, 2, 7, 32, 64, 1, 0, {64}, false},                // exactly one tile, one split
      {2, 4, 2, 4, 32, 90, 2, 16, {90, 17}, false},           // paged, the last page partly used
      {3, 2, 2, 2, 32, 48, 0, 16, {48, 1, 500}, true},        // paged, a length beyond the capacity, heuristic split count
      {2, 2, 1, 3, 32, 1100, 16, 0, {1100, 300}, false},      // nine splits: stage 2 shares each row's walk between four threads
  };
  int bad = 0;
  for (const Case& c : cases) bad += run(c);
  if (with_mfma)
    for (int late = 0; late <= (both ? 1 : 0); ++late) {
      if (host_block_loads_land_late) host_block_loads_land_late(late);
      std::printf("global->LDS loads land %s\n", late ? "late" : "when issued");
      for (const Case& c : mfma_cases) bad += run(c);
    }
  bad += run_append();
  std::printf(bad ? "FAILED\n" : "clean\n");
  return bad;
}
