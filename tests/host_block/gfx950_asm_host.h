// An interpreter for the gfx950 assembly text of the 64-row-wave loop (flash_tree_attn_amd/csrc/gen_wide_loop.py),
// so that the kernel which holds those statements runs on host threads like the rest (see hip/hip_runtime.h and
// gfx950_ops_host.h, which includes this file when the build asks for it). TEST INFRASTRUCTURE ONLY.
//
// Every host thread is one lane and interprets the statement for itself: its own copy of the vector and
// accumulation registers, and of the scalar registers, which hold the same values in all lanes of a wave. Lanes
// meet where the instruction set makes them: matrix products, the half-wave swap, the transposing LDS read and
// vector compares (whose 64-bit result every lane needs) go through the wave's exchange area, s_barrier is the
// workgroup's barrier. A statement starts from registers filled with a NaN pattern except those its operand list
// binds, so a register that the text reads without declaring it shows. The wait counters are modelled as in
// gfx950_ops_host.h: an LDS read delivers when an lgkmcnt wait lets it, and a vector instruction that names a
// register of a read still in flight aborts the run; global->LDS loads land when issued or, in the late mode, when
// a vmcnt wait forces them to; no LDS read may be in flight when the statement ends (the compiler does not know
// that the statement holds any). Instructions and operand forms: exactly those the generator emits.
#pragma once
#include <bitset>
#include <map>
#include <string>

namespace host_asm {

struct Operand {
  enum Kind { kNone, kV, kA, kS, kVcc, kM0, kLiteral, kLabel } kind = kNone;
  int lo = 0, n = 1;
  bool neg = false;
  uint32_t literal = 0;
  std::string label;
};
struct Instruction {
  std::string op, text;
  Operand o[4];
  int operands = 0;
  int offset = 0;          // ds_read: byte offset; s_nop: count
  int lgkmcnt = -1, vmcnt = -1;
  bool word1 = false;      // sdwa: the source's upper half
  std::bitset<512> names;  // vector (0..255) and accumulation (256..511) registers the instruction names
};

[[noreturn]] inline void fail(const std::string& why) {
  std::fprintf(stderr, "assembly interpreter: %s\n", why.c_str());
  std::abort();
}

inline Operand parse_operand(std::string t) {
  Operand o;
  while (!t.empty() && t.front() == ' ') t.erase(0, 1);
  while (!t.empty() && t.back() == ' ') t.pop_back();
  if (t.empty()) fail("empty operand");
  if (t == "vcc") { o.kind = Operand::kVcc; return o; }
  if (t == "m0") { o.kind = Operand::kM0; return o; }
  if (t[0] == '.') { o.kind = Operand::kLabel; o.label = t; return o; }
  if (t[0] == '-' && (t[1] == 'v' || t[1] == 'a' || t[1] == 's')) { o.neg = true; t.erase(0, 1); }
  if ((t[0] == 'v' || t[0] == 'a' || t[0] == 's') && t.size() > 1 && (t[1] == '[' || (t[1] >= '0' && t[1] <= '9'))) {
    o.kind = t[0] == 'v' ? Operand::kV : t[0] == 'a' ? Operand::kA : Operand::kS;
    int hi = 0;
    if (t[1] == '[') {
      if (std::sscanf(t.c_str() + 2, "%d:%d]", &o.lo, &hi) != 2) fail("register range `" + t + "`");
      o.n = hi - o.lo + 1;
    } else {
      o.lo = std::atoi(t.c_str() + 1);
    }
    return o;
  }
  o.kind = Operand::kLiteral;
  if (t.rfind("0x", 0) == 0) {
    o.literal = static_cast<uint32_t>(std::strtoul(t.c_str(), nullptr, 16));
  } else if (t.find('.') != std::string::npos) {
    const float f = std::strtof(t.c_str(), nullptr);   // inline float constants: 1.0, 0.5, ...
    std::memcpy(&o.literal, &f, 4);
  } else {
    o.literal = static_cast<uint32_t>(std::strtol(t.c_str(), nullptr, 10));
  }
  return o;
}

struct Program {
  std::vector<Instruction> ins;
  std::map<std::string, int> labels;
  explicit Program(const char* text) {
    std::string all(text), line;
    size_t at = 0;
    while (at < all.size()) {
      const size_t nl = all.find('\n', at);
      line = all.substr(at, nl == std::string::npos ? std::string::npos : nl - at);
      at = nl == std::string::npos ? all.size() : nl + 1;
      const size_t comment = line.find(';');
      if (comment != std::string::npos) line.erase(comment);
      while (!line.empty() && (line.back() == ' ' || line.back() == '\t')) line.pop_back();
      while (!line.empty() && (line.front() == ' ' || line.front() == '\t')) line.erase(0, 1);
      if (line.empty()) continue;
      if (line.back() == ':') { labels[line.substr(0, line.size() - 1)] = static_cast<int>(ins.size()); continue; }
      Instruction i;
      i.text = line;
      const size_t sp = line.find(' ');
      i.op = line.substr(0, sp);
      for (const char* suffix : {"_e32", "_e64"})
        if (i.op.size() > 4 && i.op.compare(i.op.size() - 4, 4, suffix) == 0) i.op.erase(i.op.size() - 4);
      std::string rest = sp == std::string::npos ? "" : line.substr(sp + 1);
      if (i.op == "s_waitcnt") {
        if (std::sscanf(rest.c_str(), " lgkmcnt(%d)", &i.lgkmcnt) != 1 && std::sscanf(rest.c_str(), " vmcnt(%d)", &i.vmcnt) != 1) fail("`" + line + "`");
      } else if (i.op == "s_nop") {
        i.offset = std::atoi(rest.c_str());
      } else if (!rest.empty()) {
        size_t start = 0;
        while (start <= rest.size()) {
          const size_t comma = rest.find(',', start);
          std::string tok = rest.substr(start, comma == std::string::npos ? std::string::npos : comma - start);
          start = comma == std::string::npos ? rest.size() + 1 : comma + 1;
          while (!tok.empty() && tok.front() == ' ') tok.erase(0, 1);
          const size_t mod = tok.find(' ');                 // modifiers behind the last operand
          if (mod != std::string::npos) {
            const std::string mods = tok.substr(mod + 1);
            tok.erase(mod);
            const size_t off = mods.find("offset:");
            if (off != std::string::npos) i.offset = static_cast<int>(std::strtol(mods.c_str() + off + 7, nullptr, 0));
            if (mods.find("src0_sel:WORD_1") != std::string::npos) i.word1 = true;
            else if (mods.find("sel:") != std::string::npos && mods.find("dst_sel:DWORD") == std::string::npos) fail("`" + line + "`");
          }
          if (i.operands == 4) fail("too many operands in `" + line + "`");
          i.o[i.operands++] = parse_operand(tok);
        }
      }
      if (i.op[0] == 'v' || i.op[0] == 'd' || i.op[0] == 'g')
        for (int k = 0; k < i.operands; ++k)
          if (i.o[k].kind == Operand::kV || i.o[k].kind == Operand::kA)
            for (int r = 0; r < i.o[k].n; ++r) i.names.set((i.o[k].kind == Operand::kA ? 256 : 0) + i.o[k].lo + r);
      ins.push_back(i);
    }
  }
};

// One operand of the statement: the register it is bound to ("v12", "a0", "s76") and the 32-bit C++ object.
struct Binding {
  const char* reg;
  uint32_t* object;
  bool written_back;   // "+" operands
};
template <typename T>
inline uint32_t* bits(const T& object) {
  static_assert(sizeof(T) == 4, "every operand is one 32-bit register");
  return reinterpret_cast<uint32_t*>(const_cast<T*>(&object));
}

struct Lane {
  uint32_t v[256], a[256], s[128];
  uint64_t vcc;
  uint32_t m0;
  bool scc;
};
struct LdsReadPending {
  int first;      // 0..255 vector, 256..511 accumulation
  int count;
  uint32_t data[4];
};

inline float as_f(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
inline uint32_t as_u(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline uint16_t bf16_rne(float f) {
  if (f != f) return 0x7FC0;
  const uint32_t u = as_u(f);
  return static_cast<uint16_t>((u + 0x7FFF + ((u >> 16) & 1)) >> 16);
}
inline float half_to_f(uint16_t h, bool bf16) {
  if (bf16) return as_f(static_cast<uint32_t>(h) << 16);
  _Float16 x;
  std::memcpy(&x, &h, 2);
  return static_cast<float>(x);
}

// Gathers one 32-bit value per lane of the wave: result[l] = what lane l passed.
inline void wave_gather(uint32_t mine, uint32_t (&all)[64]) {
  host_block::WaveExchange& x = host_block::my_exchange();
  std::memcpy(x.bytes[host_block::lane_id()], &mine, 4);
  host_wave_barrier();
  for (int l = 0; l < 64; ++l) std::memcpy(&all[l], x.bytes[l], 4);
  host_wave_barrier();
}

inline void run(const Program& prog, const Binding* bind, size_t nbind, bool bf16) {
  static thread_local Lane L;
  std::memset(&L, 0xFF, sizeof(L));
  L.scc = false;
  auto slot = [&](const char* reg) -> uint32_t& {
    const int i = std::atoi(reg + 1);
    return reg[0] == 'v' ? L.v[i] : reg[0] == 'a' ? L.a[i] : L.s[i];
  };
  for (size_t b = 0; b < nbind; ++b) slot(bind[b].reg) = *bind[b].object;
  std::deque<LdsReadPending> reads;
  std::bitset<512> in_flight;
  const unsigned lane = host_block::lane_id();

  auto vreg = [&](const Operand& o, int k = 0) -> uint32_t& { return o.kind == Operand::kA ? L.a[o.lo + k] : L.v[o.lo + k]; };
  auto src = [&](const Operand& o) -> uint32_t {
    switch (o.kind) {
      case Operand::kV: return L.v[o.lo] ^ (o.neg ? 0x80000000u : 0u);
      case Operand::kA: return L.a[o.lo] ^ (o.neg ? 0x80000000u : 0u);
      case Operand::kS: return L.s[o.lo] ^ (o.neg ? 0x80000000u : 0u);
      case Operand::kM0: return L.m0;
      case Operand::kLiteral: return o.literal;
      default: fail("operand without a 32-bit value");
    }
  };
  auto f = [&](const Operand& o) { return as_f(src(o)); };
  auto set_scalar = [&](const Operand& o, uint64_t value) {
    if (o.kind == Operand::kM0) L.m0 = static_cast<uint32_t>(value);
    else if (o.kind == Operand::kS && o.n == 1) L.s[o.lo] = static_cast<uint32_t>(value);
    else fail("scalar destination");
  };
  auto mask64 = [&](const Operand& o) -> uint64_t {
    if (o.kind == Operand::kVcc) return L.vcc;
    if (o.kind == Operand::kS && o.n == 2) return L.s[o.lo] | (static_cast<uint64_t>(L.s[o.lo + 1]) << 32);
    fail("64-bit scalar operand");
  };
  auto set_mask64 = [&](const Operand& o, uint64_t bitsv) {
    if (o.kind == Operand::kVcc) L.vcc = bitsv;
    else if (o.kind == Operand::kS && o.n == 2) { L.s[o.lo] = static_cast<uint32_t>(bitsv); L.s[o.lo + 1] = static_cast<uint32_t>(bitsv >> 32); }
    else fail("64-bit scalar destination");
  };
  auto jump = [&](const Operand& o) -> int {
    auto it = prog.labels.find(o.label);
    if (it == prog.labels.end()) fail("label " + o.label);
    return it->second;
  };

  size_t pc = 0, executed = 0;
  while (pc < prog.ins.size()) {
    const Instruction& i = prog.ins[pc++];
    const std::string& op = i.op;
    if (++executed > 50'000'000) fail("statement does not end");
    if (op == "s_nop") continue;
    if (op == "s_waitcnt") {
      if (i.lgkmcnt >= 0)
        while (reads.size() > static_cast<size_t>(i.lgkmcnt)) {
          const LdsReadPending& r = reads.front();
          for (int k = 0; k < r.count; ++k) {
            (r.first >= 256 ? L.a[r.first - 256 + k] : L.v[r.first + k]) = r.data[k];
            in_flight.reset(r.first + k);
          }
          reads.pop_front();
        }
      if (i.vmcnt >= 0) host_block::land_all_but(static_cast<size_t>(i.vmcnt));
      continue;
    }
    if ((i.names & in_flight).any()) fail("`" + i.text + "` names a register of an LDS read that no lgkmcnt wait has covered");
    const Operand *o = i.o;
    if (op == "s_barrier") {
      host_block::current()->all.arrive_and_wait();
    } else if (op == "s_branch") {
      pc = jump(o[0]);
    } else if (op == "s_cbranch_scc1") {
      if (L.scc) pc = jump(o[0]);
    } else if (op == "s_cbranch_vccnz") {
      if (L.vcc != 0) pc = jump(o[0]);
    } else if (op == "s_cbranch_vccz") {
      if (L.vcc == 0) pc = jump(o[0]);
    } else if (op == "s_mov_b32") {
      set_scalar(o[0], src(o[1]));
    } else if (op == "s_mov_b64") {
      set_mask64(o[0], mask64(o[1]));
    } else if (op == "s_or_b64" || op == "s_and_b64") {
      const uint64_t r = op == "s_or_b64" ? (mask64(o[1]) | mask64(o[2])) : (mask64(o[1]) & mask64(o[2]));
      set_mask64(o[0], r);
      L.scc = r != 0;
    } else if (op == "s_add_u32") {
      const uint64_t r = static_cast<uint64_t>(src(o[1])) + src(o[2]);
      L.scc = r > 0xFFFFFFFFull;
      set_scalar(o[0], r);
    } else if (op == "s_addc_u32") {
      const uint64_t r = static_cast<uint64_t>(src(o[1])) + src(o[2]) + (L.scc ? 1 : 0);
      L.scc = r > 0xFFFFFFFFull;
      set_scalar(o[0], r);
    } else if (op == "s_sub_u32") {
      const uint32_t x = src(o[1]), y = src(o[2]);
      L.scc = y > x;
      set_scalar(o[0], x - y);
    } else if (op == "s_cmp_eq_u32") {
      L.scc = src(o[0]) == src(o[1]);
    } else if (op == "s_cmp_lg_u32") {
      L.scc = src(o[0]) != src(o[1]);
    } else if (op == "s_cmp_gt_u32") {
      L.scc = src(o[0]) > src(o[1]);
    } else if (op == "s_cselect_b32") {
      set_scalar(o[0], L.scc ? src(o[1]) : src(o[2]));
    } else if (op == "v_mov_b32" || op == "v_accvgpr_read_b32" || op == "v_accvgpr_write_b32") {
      vreg(o[0]) = src(o[1]);
    } else if (op == "v_add_u32") {
      vreg(o[0]) = src(o[1]) + src(o[2]);
    } else if (op == "v_lshlrev_b32") {
      vreg(o[0]) = src(o[2]) << (src(o[1]) & 31);
    } else if (op == "v_and_b32") {
      vreg(o[0]) = src(o[1]) & src(o[2]);
    } else if (op == "v_add_f32") {
      vreg(o[0]) = as_u(f(o[1]) + f(o[2]));
    } else if (op == "v_sub_f32") {
      vreg(o[0]) = as_u(f(o[1]) - f(o[2]));
    } else if (op == "v_mul_f32") {
      vreg(o[0]) = as_u(f(o[1]) * f(o[2]));
    } else if (op == "v_fma_f32") {
      vreg(o[0]) = as_u(std::fmaf(f(o[1]), f(o[2]), f(o[3])));
    } else if (op == "v_max_f32") {
      vreg(o[0]) = as_u(std::fmaxf(f(o[1]), f(o[2])));
    } else if (op == "v_max3_f32") {
      vreg(o[0]) = as_u(std::fmaxf(std::fmaxf(f(o[1]), f(o[2])), f(o[3])));
    } else if (op == "v_exp_f32") {
      vreg(o[0]) = as_u(static_cast<float>(std::exp2(static_cast<double>(f(o[1])))));
    } else if (op == "v_cmp_neq_f32" || op == "v_cmp_nge_f32") {
      if (o[0].kind != Operand::kVcc) fail("`" + i.text + "`");
      const bool mine = op == "v_cmp_neq_f32" ? !(f(o[1]) == f(o[2])) : !(f(o[1]) >= f(o[2]));
      uint32_t all[64];
      wave_gather(mine ? 1u : 0u, all);
      L.vcc = 0;
      for (int l = 0; l < 64; ++l) L.vcc |= static_cast<uint64_t>(all[l] & 1) << l;
    } else if (op == "v_cndmask_b32") {
      if (o[3].kind != Operand::kVcc) fail("`" + i.text + "`");
      vreg(o[0]) = (L.vcc >> lane) & 1 ? src(o[2]) : src(o[1]);
    } else if (op == "v_cvt_pk_bf16_f32") {
      vreg(o[0]) = bf16_rne(f(o[1])) | (static_cast<uint32_t>(bf16_rne(f(o[2]))) << 16);
    } else if (op == "v_cvt_pk_f16_f32") {
      const _Float16 lo = static_cast<_Float16>(f(o[1])), hi = static_cast<_Float16>(f(o[2]));
      uint16_t l16, h16;
      std::memcpy(&l16, &lo, 2);
      std::memcpy(&h16, &hi, 2);
      vreg(o[0]) = l16 | (static_cast<uint32_t>(h16) << 16);
    } else if (op == "v_dot2c_f32_bf16" || op == "v_dot2c_f32_f16") {
      const bool b16 = op == "v_dot2c_f32_bf16";
      const uint32_t x = src(o[1]), y = src(o[2]);
      const double acc = static_cast<double>(as_f(vreg(o[0]))) +
                         static_cast<double>(half_to_f(x & 0xFFFF, b16)) * half_to_f(y & 0xFFFF, b16) +
                         static_cast<double>(half_to_f(x >> 16, b16)) * half_to_f(y >> 16, b16);
      vreg(o[0]) = as_u(static_cast<float>(acc));
    } else if (op == "v_cvt_f32_f16" || op == "v_cvt_f32_f16_sdwa") {
      const uint32_t x = src(o[1]);
      vreg(o[0]) = as_u(half_to_f(static_cast<uint16_t>(op == "v_cvt_f32_f16_sdwa" && i.word1 ? x >> 16 : x & 0xFFFF), false));
      if (op == "v_cvt_f32_f16_sdwa" && !i.word1) fail("`" + i.text + "`");
    } else if (op == "v_permlane32_swap_b32") {
      // the upper half of the first register trades places with the lower half of the second
      host_block::WaveExchange& x = host_block::my_exchange();
      const uint32_t pair[2] = {vreg(o[0]), vreg(o[1])};
      std::memcpy(x.bytes[lane], pair, 8);
      host_wave_barrier();
      uint32_t other[2];
      std::memcpy(other, x.bytes[lane ^ 32], 8);
      host_wave_barrier();
      if (lane < 32) vreg(o[1]) = other[0]; else vreg(o[0]) = other[1];
    } else if (op == "v_mfma_f32_32x32x16_bf16" || op == "v_mfma_f32_32x32x16_f16") {
      if ((op == "v_mfma_f32_32x32x16_bf16") != bf16 || o[0].n != 16 || o[1].n != 4 || o[2].n != 4) fail("`" + i.text + "`");
      uint32_t ar[4], br[4];
      for (int k = 0; k < 4; ++k) { ar[k] = vreg(o[1], k); br[k] = vreg(o[2], k); }
      fta::f32x16 c;
      for (int k = 0; k < 16; ++k) c[k] = o[3].kind == Operand::kLiteral ? as_f(o[3].literal) : as_f(vreg(o[3], k));
      fta::f32x16 d;
      if (bf16) {
        fta::bf16x8 av, bv;
        std::memcpy(&av, ar, 16);
        std::memcpy(&bv, br, 16);
        d = fta::host_mfma_32x32x16(av, bv, c);
      } else {
        fta::f16x8 av, bv;
        std::memcpy(&av, ar, 16);
        std::memcpy(&bv, br, 16);
        d = fta::host_mfma_32x32x16(av, bv, c);
      }
      for (int k = 0; k < 16; ++k) vreg(o[0], k) = as_u(d[k]);
    } else if (op == "ds_read_b128" || op == "ds_read_b64_tr_b16") {
      const uint32_t addr = src(o[1]) + static_cast<uint32_t>(i.offset);
      LdsReadPending r;
      r.first = (o[0].kind == Operand::kA ? 256 : 0) + o[0].lo;
      if (op == "ds_read_b128") {
        if (o[0].n != 4) fail("`" + i.text + "`");
        r.count = 4;
        std::memcpy(r.data, host_block::lds_at(addr, 16), 16);
      } else {
        if (o[0].n != 2) fail("`" + i.text + "`");
        r.count = 2;
        host_block::WaveExchange& x = host_block::my_exchange();
        const unsigned s = lane & 15, group = lane & ~15u;
        std::memcpy(x.bytes[lane], host_block::lds_at(addr, 8), 8);
        host_wave_barrier();
        uint16_t out[4];
        for (unsigned e = 0; e < 4; ++e) std::memcpy(&out[e], x.bytes[group + 4 * e + s / 4] + 2 * (s % 4), 2);
        host_wave_barrier();
        std::memcpy(r.data, out, 8);
      }
      for (int k = 0; k < r.count; ++k) {
        (r.first >= 256 ? L.a[r.first - 256 + k] : L.v[r.first + k]) = 0xFFFFFFFFu;
        in_flight.set(r.first + k);
      }
      reads.push_back(r);
    } else if (op == "global_load_lds_dwordx4") {
      if (o[1].kind != Operand::kS || o[1].n != 2) fail("`" + i.text + "`");
      const uint64_t base = L.s[o[1].lo] | (static_cast<uint64_t>(L.s[o[1].lo + 1]) << 32);
      const char* from = reinterpret_cast<const char*>(base + src(o[0]));
      const uint32_t to = L.m0 + 16 * lane;
      if (host_block::loads_land_late()) {
        (void)host_block::lds_at(to, 16);
        host_block::loads_in_flight().push_back({from, to});
      } else {
        std::memcpy(host_block::lds_at(to, 16), from, 16);
      }
    } else {
      fail("no such instruction here: `" + i.text + "`");
    }
  }
  if (!reads.empty()) fail("the statement ends with LDS reads in flight");
  for (size_t b = 0; b < nbind; ++b)
    if (bind[b].written_back) *bind[b].object = slot(bind[b].reg);
}

}  // namespace host_asm
