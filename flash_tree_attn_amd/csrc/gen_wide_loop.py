"""Generates wide_loop_asm.inc: the hand-scheduled gfx950 assembly of the half-tile pipeline
of the stage-1 MFMA kernel (4 waves x 64 query rows, one wave per SIMD).

Why assembly: the loop keeps about 350 registers live per lane (O 128, Q 64, scores 64,
probabilities 32, operand fragments 32, ...). hipcc places them over 512 registers but, under
that pressure, parks parts of the accumulators in ordinary registers, renames them between the
two roles of the loop and spills the Q fragments to scratch; each costs more than the loop's own
vector work. Here every value has one fixed register for the whole loop.

Run `python gen_wide_loop.py` (no arguments) to rewrite wide_loop_asm.inc next to this file; the
build does so before compiling, and tests/test_kernel_asm.py checks that the committed file is
what this script produces.

The loop (one iteration = one full 64-key cache tile t, two steps of 32 keys):
  step 0:  matrix: S[1] = K(t, keys 32..63) . Q^T ;  O += V(t-1, keys 32..63)^T . P[2..3]
           vector: P[0..1] = exp2(S[0] * c - m)          (scores of keys 0..31 of tile t)
  sync:    wait for this wave's share of tile t+1, barrier, request tile t+4 into the stages
           of K(t) and V(t-1), which every wave has finished reading
  step 1:  matrix: S[0] = K(t+1, keys 0..31) . Q^T ;  O += V(t, keys 0..31)^T . P[0..1]
           vector: P[2..3] = exp2(S[1] * c - m)
The softmax is lazy: m is the running reference, not the running maximum, and is only raised when
a lane's probabilities of one step add up to more than LIMIT (or are not finite): that step is then
redone exactly (row maximum, rescaling of l and O) in an out-of-line block. See
stage1_mfma_kernel.h for the surrounding kernel and the meaning of every operand.
"""
from __future__ import annotations

import os

NW = 4          # waves per workgroup
NSK, NSV = 4, 5  # ring depths (tiles)
PF = 4          # operand fragments requested ahead of the MFMA that consumes them


LIMIT = 4096.0  # a step whose probabilities sum to more than this in one lane is redone exactly (every value stays representable in f16)

# ---- register map (must match the operand constraints emitted below) -------------------
A_O = 0          # a[0:127]   O^T accumulators, o[db][qb] at 16 * (db * 2 + qb)
A_Q = 128        # a[128:191] Q fragments, qf[qb][ks] at 4 * (qb * KS + ks)
V_S = 64         # v[64:127]  scores, s[h][qb] at 16 * (h * 2 + qb)
V_P = 128        # v[128:159] packed probabilities, p[qb][kk] at 4 * (qb * 4 + kk)
V_KF = 160       # v[160:175] K fragment queue (PF x 128 bit)
V_VF = 176       # v[176:191] V^T fragment queue (PF x 2 x 64 bit)
V_M = 192        # v192, v193 reference m per row block
V_L = 194        # v194, v195 running sum l per row block
V_KRD, V_VRD = 196, 197      # per-lane LDS read bases
V_KOFF, V_VOFF = 198, 199    # per-lane global byte offsets of the tile loads
V_PS = 200       # v200..v203 partial sums ps0[qb], ps1[qb]
V_E = 204        # v204..v211 exp staging (two sets, alternating by fragment)
V_KA0, V_KA1, V_VA = 212, 213, 214   # LDS addresses of the K reads of step 0 / step 1 and of this step's V reads
V_T = 215        # v215..v220 temporaries of the exact redo
V_MADD = 16      # v16..v47  masked step: additive term per score (mask * log2 e, -inf past the key limit), [qb][16]
V_R = 48         # v48..v63  masked step: packed rounding residue of P, [qb][2][2 words... 4 per 16 keys]
S_KRUN, S_VRUN = 64, 66      # s[64:65], s[66:67] global address of the next tile to request (this wave's first block)
S_KSTEP, S_VSTEP = 68, 70    # bytes between this wave's consecutive blocks of a tile (64 bit)
S_KTILE, S_VTILE = 72, 74    # bytes between tiles (64 bit)
S_KCUR, S_KNEXT, S_VPREV, S_VCUR, S_PVOFF = 76, 77, 78, 79, 80   # ring stage byte offsets
S_KDST, S_VDST = 81, 82      # LDS address of this wave's first block in stage 0 of the K / V ring
S_NT, S_NREAL, S_C = 83, 84, 85
S_TMP = 86       # s86..s93 temporaries


def layout(D: int):
    row = 2 * D
    rpb = 1024 // row
    chunk = 16 * rpb
    pitch = 1024 + chunk
    blocks = 64 // rpb
    tile = blocks * pitch
    return dict(rpb=rpb, chunk=chunk, pitch=pitch, blocks=blocks, tile=tile,
                kb_off=(32 // rpb) * pitch, ks_off=2 * chunk,
                v8=(8 // rpb) * pitch + (8 % rpb) * 16, v16=(16 // rpb) * pitch,
                loads=blocks // NW)


def gen(D: int, dtype: str) -> list[str]:
    L = layout(D)
    KS, DB = D // 16, D // 32
    NSTEP = KS + 2 * DB
    PPS = (16 + NSTEP - 1) // NSTEP
    mfma = "v_mfma_f32_32x32x16_bf16" if dtype == "bf16" else "v_mfma_f32_32x32x16_f16"
    cvt = "v_cvt_pk_bf16_f32" if dtype == "bf16" else "v_cvt_pk_f16_f32"
    dot = "v_dot2c_f32_bf16_e32" if dtype == "bf16" else "v_dot2c_f32_f16_e32"
    ones = "0x3f803f80" if dtype == "bf16" else "0x3c003c00"
    out: list[str] = []

    e = out.append

    def vr(base, n=1):
        return f"v{base}" if n == 1 else f"v[{base}:{base + n - 1}]"

    def ar(base, n=1):
        return f"a{base}" if n == 1 else f"a[{base}:{base + n - 1}]"

    def s_reg(h, qb, r=None):
        base = V_S + 16 * (h * 2 + qb)
        return vr(base, 16) if r is None else vr(base + r)

    def p_reg(qb, kk, w=None):
        base = V_P + 4 * (qb * 4 + kk)
        return vr(base, 4) if w is None else vr(base + w)

    def frag_weight(i):      # LDS reads of fragment i of a step (K: one 128-bit read, V: two 64-bit)
        return 1 if i < KS else 2

    def issue_frag(i, ka, va=V_VA):
        if i < KS:
            e(f"ds_read_b128 {vr(V_KF + 4 * (i % PF), 4)}, v{ka} offset:{i * L['ks_off']}")
        else:
            g = i - KS
            off = (g // DB) * L["v16"] + (g % DB) * 4 * L["chunk"]
            base = V_VF + 4 * (g % PF)
            e(f"ds_read_b64_tr_b16 {vr(base, 2)}, v{va} offset:{off}")
            e(f"ds_read_b64_tr_b16 {vr(base + 2, 2)}, v{va} offset:{off + L['v8']}")

    def pair_regs(H, j):
        qb, jj = j // 8, j % 8
        r = 2 * jj
        return qb, s_reg(H, qb, r), s_reg(H, qb, r + 1), p_reg(qb, 2 * H + (1 if jj >= 4 else 0), jj % 4)

    def step(H, cross_prefetch, extra=()):
        """One half-tile step. K fragments 0..PF-1 have been requested already. With
        cross_prefetch the first PF K fragments of the NEXT step (H' = 0, next tile) are
        requested during the last fragments of this one. `extra`: groups of scalar / load
        instructions (the tile request) to spread over the fragments, one group each."""
        e(f"; ---- step {H}")
        for r in range(4):
            e(f"v_mov_b32 {vr(V_PS + r)}, 0")
        pending = []   # (cvt, dot) instructions of the previous fragment's pairs
        extra = list(extra)
        for i in range(NSTEP):
            # reads queued behind fragment i: fragments i+1 .. i+PF-1 of the stream
            newer = 0
            for k in range(i + 1, i + PF):
                if k < NSTEP:
                    newer += frag_weight(k)
                elif cross_prefetch:
                    newer += 1   # a K fragment of the next step
            valu = []
            for j in range(i * PPS, min(16, (i + 1) * PPS)):
                qb, s0, s1, pdst = pair_regs(H, j)
                e0 = V_E + 2 * ((j - i * PPS) + PPS * (i % 2))
                valu.append((f"v_fma_f32 {vr(e0)}, {s0}, s{S_C}, -{vr(V_M + qb)}",
                             f"v_fma_f32 {vr(e0 + 1)}, {s1}, s{S_C}, -{vr(V_M + qb)}",
                             f"v_exp_f32_e32 {vr(e0)}, {vr(e0)}",
                             f"v_exp_f32_e32 {vr(e0 + 1)}, {vr(e0 + 1)}",
                             f"{cvt} {pdst}, {vr(e0)}, {vr(e0 + 1)}",
                             f"{dot} {vr(V_PS + 2 * qb + (j & 1))}, {ones}, {pdst}"))
            # the two MFMAs of the fragment, each followed by about half of the other work
            mark = len(out)
            if i + PF < NSTEP:
                issue_frag(i + PF, V_KA0 if H == 0 else V_KA1)
            elif cross_prefetch:
                issue_frag(i + PF - NSTEP, V_KA0)   # step 0 of the next tile: its address is already in place
            reads = out[mark:]
            del out[mark:]
            # (the reads overwrite the fragment both MFMAs use: they go behind the second one)
            slot_a = [x for v in valu for x in (v[0], v[1])] + [x for v in valu for x in (v[2], v[3])]
            slot_b = reads + pending + (extra.pop(0) if extra else [])
            mm = []
            for qb in range(2):
                if i < KS:
                    a = vr(V_KF + 4 * (i % PF), 4)
                    b = ar(A_Q + 4 * (qb * KS + i), 4)
                    cd = s_reg(1 - H, qb)
                    mm.append(f"{mfma} {cd}, {a}, {b}, {'0' if i == 0 else cd}")
                else:
                    g = i - KS
                    a = vr(V_VF + 4 * (g % PF), 4)
                    b = p_reg(qb, 2 * (1 - H) + g // DB)
                    cd = ar(A_O + 16 * ((g % DB) * 2 + qb), 16)
                    mm.append(f"{mfma} {cd}, {a}, {b}, {cd}")
            e(f"s_waitcnt lgkmcnt({newer})")
            e(mm[0])
            for ins in slot_a:
                e(ins)
            e(mm[1])
            for ins in slot_b:
                e(ins)
            pending = [x for v in valu for x in (v[4], v[5])]
        assert not extra, "more request groups than fragments"
        for ins in pending:
            e(ins)
        # lazy-softmax check: any lane whose probabilities of this step sum to more than LIMIT, or to a non-number
        t0, t1 = V_E, V_E + 1
        e("s_nop 3")   # a dot instruction's result may be read by another kind of instruction only 3 issue cycles later (no interlock)
        e(f"v_add_f32 {vr(t0)}, {vr(V_PS)}, {vr(V_PS + 1)}")
        e(f"v_add_f32 {vr(t1)}, {vr(V_PS + 2)}, {vr(V_PS + 3)}")
        e(f"v_cmp_nge_f32_e32 vcc, 0x{_f32(LIMIT)}, {vr(t0)}")     # !(LIMIT >= sum): larger, or not a number
        e(f"s_mov_b64 s[{S_TMP + 4}:{S_TMP + 5}], vcc")
        e(f"v_cmp_nge_f32_e32 vcc, 0x{_f32(LIMIT)}, {vr(t1)}")
        e(f"s_or_b64 vcc, vcc, s[{S_TMP + 4}:{S_TMP + 5}]")
        e(f"s_cbranch_vccnz .Lfix{H}_%=")
        e(f"v_add_f32 {vr(V_L)}, {vr(V_L)}, {vr(t0)}")
        e(f"v_add_f32 {vr(V_L + 1)}, {vr(V_L + 1)}, {vr(t1)}")
        e(f".Ldone{H}_%=:")

    def fix(H):
        """Exact redo of step H from its scores (still in s[H]): raise m to the true maximum,
        rescale l and O, rebuild P[2H..2H+1], add the new sums to l."""
        e(f".Lfix{H}_%=:")
        e("s_nop 15")   # the P.V products issued last must have left the matrix pipeline before O is read
        e("s_nop 15")
        e("s_nop 15")
        t = V_T
        for qb in range(2):
            sr = [s_reg(H, qb, r) for r in range(16)]
            e(f"v_max3_f32 {vr(t)}, {sr[0]}, {sr[1]}, {sr[2]}")
            for r in range(3, 15, 2):
                e(f"v_max3_f32 {vr(t)}, {vr(t)}, {sr[r]}, {sr[r + 1]}")
            e(f"v_max_f32 {vr(t)}, {vr(t)}, {sr[15]}")
            e(f"v_mov_b32 {vr(t + 1)}, {vr(t)}")
            e("s_nop 1")
            e(f"v_permlane32_swap_b32 {vr(t)}, {vr(t + 1)}")   # lanes < 32: partner in t+1; lanes >= 32: partner in t
            e("s_nop 1")
            e(f"v_max_f32 {vr(t)}, {vr(t)}, {vr(t + 1)}")
            e(f"v_mul_f32 {vr(t)}, s{S_C}, {vr(t)}")
            e(f"v_max_f32 {vr(t + 2)}, {vr(V_M + qb)}, {vr(t)}")             # m_new
            e(f"v_sub_f32 {vr(t + 3)}, {vr(V_M + qb)}, {vr(t + 2)}")
            e(f"v_exp_f32_e32 {vr(t + 3)}, {vr(t + 3)}")                     # alpha = 2^(m - m_new); 0 for m = -inf
            e(f"v_mov_b32 {vr(V_M + qb)}, {vr(t + 2)}")
            e(f"v_mov_b32 {vr(t + 4)}, 0")
            e(f"v_mul_f32 {vr(V_L + qb)}, {vr(V_L + qb)}, {vr(t + 3)}")
            for jj in range(8):
                r = 2 * jj
                pdst = p_reg(qb, 2 * H + (1 if jj >= 4 else 0), jj % 4)
                e(f"v_fma_f32 {vr(V_E)}, {sr[r]}, s{S_C}, -{vr(V_M + qb)}")
                e(f"v_fma_f32 {vr(V_E + 1)}, {sr[r + 1]}, s{S_C}, -{vr(V_M + qb)}")
                e(f"v_exp_f32_e32 {vr(V_E)}, {vr(V_E)}")
                e(f"v_exp_f32_e32 {vr(V_E + 1)}, {vr(V_E + 1)}")
                e("s_nop 0")
                e(f"{cvt} {pdst}, {vr(V_E)}, {vr(V_E + 1)}")
                e(f"{dot} {vr(t + 4)}, {ones}, {pdst}")
            e("s_nop 3")   # dot result -> other instruction: 3 idle issue cycles
            e(f"v_add_f32 {vr(V_L + qb)}, {vr(V_L + qb)}, {vr(t + 4)}")
            for db in range(DB):
                base = A_O + 16 * (db * 2 + qb)
                for r in range(16):
                    e(f"v_accvgpr_read_b32 {vr(t + 5)}, {ar(base + r)}")
                    e(f"v_mul_f32 {vr(t + 5)}, {vr(t + 5)}, {vr(t + 3)}")
                    e(f"v_accvgpr_write_b32 {ar(base + r)}, {vr(t + 5)}")
        e("s_nop 7")
        e(f"s_branch .Ldone{H}_%=")

    S_KLDS, S_VLDS = S_TMP + 6, S_TMP + 7   # LDS addresses of this request's first K / V block (taken before the ring advances)

    def request_groups():
        """The loads of one tile into the K stage of tile t and the V stage of tile t-1, as
        groups of instructions (one load each) for step 1 to spread over its fragments. While
        real tiles remain the global addresses advance; afterwards the last tile is requested
        again (into a stage nobody reads) so that every synchronisation point has the same
        number of loads in flight."""
        groups = []
        for (run, stepr, lds, voff) in ((S_KRUN, S_KSTEP, S_KLDS, V_KOFF), (S_VRUN, S_VSTEP, S_VLDS, V_VOFF)):
            for i in range(L["loads"]):
                g = []
                if i == 0:
                    g.append(f"s_mov_b64 s[{S_TMP}:{S_TMP + 1}], s[{run}:{run + 1}]")
                    g.append(f"s_mov_b32 m0, s{lds}")
                else:
                    g.append(f"s_add_u32 s{S_TMP}, s{S_TMP}, s{stepr}")
                    g.append(f"s_addc_u32 s{S_TMP + 1}, s{S_TMP + 1}, s{stepr + 1}")
                    g.append(f"s_add_u32 m0, m0, {NW * L['pitch']}")
                g.append("s_nop 0")
                g.append(f"global_load_lds_dwordx4 v{voff}, s[{S_TMP}:{S_TMP + 1}]")
                groups.append(g)
        adv = [f"s_cmp_gt_u32 s{S_NREAL}, 1",
               # all four selects before the first add: the adds overwrite the condition bit
               f"s_cselect_b32 s{S_TMP}, s{S_KTILE}, 0", f"s_cselect_b32 s{S_TMP + 1}, s{S_KTILE + 1}, 0",
               f"s_cselect_b32 s{S_TMP + 2}, s{S_VTILE}, 0", f"s_cselect_b32 s{S_TMP + 3}, s{S_VTILE + 1}, 0",
               f"s_add_u32 s{S_KRUN}, s{S_KRUN}, s{S_TMP}", f"s_addc_u32 s{S_KRUN + 1}, s{S_KRUN + 1}, s{S_TMP + 1}",
               f"s_add_u32 s{S_VRUN}, s{S_VRUN}, s{S_TMP + 2}", f"s_addc_u32 s{S_VRUN + 1}, s{S_VRUN + 1}, s{S_TMP + 3}",
               f"s_cmp_lg_u32 s{S_NREAL}, 0", f"s_cselect_b32 s{S_TMP + 2}, 1, 0", f"s_sub_u32 s{S_NREAL}, s{S_NREAL}, s{S_TMP + 2}"]
        groups.append(adv)
        return groups

    # ---- entry: S[0] = K(first tile, keys 0..31) . Q^T, P[.][2..3] = 0 (the first step's P.V adds nothing)
    for qb in range(2):
        for kk in (2, 3):
            for w in range(4):
                e(f"v_mov_b32 {p_reg(qb, kk, w)}, 0")
    e(f"v_add_u32 v{V_KA1}, s{S_KCUR}, v{V_KRD}")
    for i in range(min(PF, KS)):
        issue_frag(i, V_KA1)
    for i in range(KS):
        e(f"s_waitcnt lgkmcnt({min(PF - 1, KS - 1 - i)})")
        for qb in range(2):
            cd = s_reg(0, qb)
            e(f"{mfma} {cd}, {vr(V_KF + 4 * (i % PF), 4)}, {ar(A_Q + 4 * (qb * KS + i), 4)}, {'0' if i == 0 else cd}")
        if i + PF < KS:
            issue_frag(i + PF, V_KA1)
    # addresses and first K fragments of step 0 of the first tile
    e(f"s_add_u32 s{S_TMP + 2}, s{S_KCUR}, {L['kb_off']}")
    e(f"v_add_u32 v{V_KA0}, s{S_TMP + 2}, v{V_KRD}")
    for i in range(PF):
        issue_frag(i, V_KA0)
    e("s_nop 15")   # the scores just computed are read by the vector ALU next: let the last MFMAs retire
    e("s_nop 15")
    e(".Lloop_%=:")
    # step 0: scores of keys 32..63 of tile t from K stage kcur, P.V of keys 32..63 of tile t-1 from pvoff
    e(f"v_add_u32 v{V_VA}, s{S_PVOFF}, v{V_VRD}")
    step(0, cross_prefetch=False)
    # synchronisation point
    e(f"s_waitcnt vmcnt({2 * 2 * L['loads']})")
    e("s_barrier")
    e(f"v_add_u32 v{V_KA1}, s{S_KNEXT}, v{V_KRD}")   # step 1 reads keys 0..31 of tile t+1
    e(f"v_add_u32 v{V_VA}, s{S_VCUR}, v{V_VRD}")    # and V rows 0..31 of tile t
    for i in range(PF):
        issue_frag(i, V_KA1)
    e(f"s_add_u32 s{S_KLDS}, s{S_KDST}, s{S_KCUR}")    # where the tile requested during step 1 lands
    e(f"s_add_u32 s{S_VLDS}, s{S_VDST}, s{S_VPREV}")
    # ring bookkeeping for the next tile
    e(f"s_mov_b32 s{S_VPREV}, s{S_VCUR}")
    e(f"s_add_u32 s{S_VCUR}, s{S_VCUR}, {L['tile']}")
    e(f"s_cmp_eq_u32 s{S_VCUR}, {NSV * L['tile']}")
    e(f"s_cselect_b32 s{S_VCUR}, 0, s{S_VCUR}")
    e(f"s_mov_b32 s{S_KCUR}, s{S_KNEXT}")
    e(f"s_add_u32 s{S_KNEXT}, s{S_KNEXT}, {L['tile']}")
    e(f"s_cmp_eq_u32 s{S_KNEXT}, {NSK * L['tile']}")
    e(f"s_cselect_b32 s{S_KNEXT}, 0, s{S_KNEXT}")
    e(f"s_add_u32 s{S_PVOFF}, s{S_VPREV}, {2 * L['v16']}")
    # address of the next tile's step-0 K reads (keys 32..63 of tile t+1, now `kcur`), for the prefetch across the loop edge
    e(f"s_add_u32 s{S_TMP + 2}, s{S_KCUR}, {L['kb_off']}")
    e(f"v_add_u32 v{V_KA0}, s{S_TMP + 2}, v{V_KRD}")
    step(1, cross_prefetch=True, extra=request_groups())
    e(f"s_sub_u32 s{S_NT}, s{S_NT}, 1")
    e(f"s_cmp_lg_u32 s{S_NT}, 0")
    e(f"s_cbranch_scc1 .Lloop_%=")
    # ---- exit: the P.V product still owed, O += V(last tile, keys 32..63)^T . P[2..3] (what step 0 of a next tile would do)
    e(f"v_add_u32 v{V_VA}, s{S_PVOFF}, v{V_VRD}")
    NV = 2 * DB
    for g in range(min(PF, NV)):
        issue_frag(KS + g, V_KA0)
    for g in range(NV):
        e(f"s_waitcnt lgkmcnt({2 * min(PF - 1, NV - 1 - g)})")
        for qb in range(2):
            cd = ar(A_O + 16 * ((g % DB) * 2 + qb), 16)
            e(f"{mfma} {cd}, {vr(V_VF + 4 * (g % PF), 4)}, {p_reg(qb, 2 + g // DB)}, {cd}")
        if g + PF < NV:
            issue_frag(KS + g + PF, V_KA0)
    e(f"s_branch .Lend_%=")
    fix(0)
    fix(1)
    e(".Lend_%=:")
    e("s_nop 15")   # the compiler does not know that MFMAs came last: let them retire before it touches O
    return out


def gen_masked(D: int, dtype: str, H: int) -> list[str]:
    """One masked half tile (32 keys of a tree tile or of the ragged last cache tile), complete:
    scores, additive term, exact online softmax (l and O rescaled at once), P.V and the
    compensating P.V product with the rounding residue of P. Same register map as the loop;
    the K / V stage offsets of the half come in s76 / s79."""
    L = layout(D)
    KS, DB = D // 16, D // 32
    mfma = "v_mfma_f32_32x32x16_bf16" if dtype == "bf16" else "v_mfma_f32_32x32x16_f16"
    cvt = "v_cvt_pk_bf16_f32" if dtype == "bf16" else "v_cvt_pk_f16_f32"
    out: list[str] = []
    e = out.append

    def vr(base, n=1):
        return f"v{base}" if n == 1 else f"v[{base}:{base + n - 1}]"

    def ar(base, n=1):
        return f"a{base}" if n == 1 else f"a[{base}:{base + n - 1}]"

    def s_reg(qb, r=None):
        base = V_S + 16 * (H * 2 + qb)
        return vr(base, 16) if r is None else vr(base + r)

    def p_word(qb, kk, w):      # kk: 0, 1 within the half
        return V_P + 4 * (qb * 4 + 2 * H + kk) + w

    def r_word(qb, kk, w):
        return V_R + 4 * (qb * 2 + kk) + w

    KA, VA = V_KA0, V_VA
    t = V_T
    NV = 2 * DB
    # ---- scores S[H] = K(half) . Q^T
    e(f"v_add_u32 v{KA}, s{S_KCUR}, v{V_KRD}")
    e(f"v_add_u32 v{VA}, s{S_VCUR}, v{V_VRD}")
    for i in range(min(PF, KS)):
        e(f"ds_read_b128 {vr(V_KF + 4 * (i % PF), 4)}, v{KA} offset:{i * L['ks_off']}")
    for i in range(KS):
        e(f"s_waitcnt lgkmcnt({min(PF - 1, KS - 1 - i)})")
        for qb in range(2):
            cd = s_reg(qb)
            e(f"{mfma} {cd}, {vr(V_KF + 4 * (i % PF), 4)}, {ar(A_Q + 4 * (qb * KS + i), 4)}, {'0' if i == 0 else cd}")
        if i + PF < KS:
            e(f"ds_read_b128 {vr(V_KF + 4 * (i % PF), 4)}, v{KA} offset:{(i + PF) * L['ks_off']}")

    def issue_v(g):
        off = (g // DB) * L["v16"] + (g % DB) * 4 * L["chunk"]
        base = V_VF + 4 * (g % PF)
        e(f"ds_read_b64_tr_b16 {vr(base, 2)}, v{VA} offset:{off}")
        e(f"ds_read_b64_tr_b16 {vr(base + 2, 2)}, v{VA} offset:{off + L['v8']}")

    for g in range(min(PF, NV)):     # V^T fragments on their way while the softmax runs
        issue_v(g)
    e("s_nop 15")   # the scores are read by the vector ALU next: let the last MFMAs retire
    e("s_nop 15")
    e("s_nop 15")
    # ---- exact online softmax per row block
    for qb in range(2):
        sr = [s_reg(qb, r) for r in range(16)]
        for r in range(16):
            e(f"v_fma_f32 {sr[r]}, {sr[r]}, s{S_C}, {vr(V_MADD + 16 * qb + r)}")
        e(f"v_max3_f32 {vr(t)}, {sr[0]}, {sr[1]}, {sr[2]}")
        for r in range(3, 15, 2):
            e(f"v_max3_f32 {vr(t)}, {vr(t)}, {sr[r]}, {sr[r + 1]}")
        e(f"v_max_f32 {vr(t)}, {vr(t)}, {sr[15]}")
        e(f"v_mov_b32 {vr(t + 1)}, {vr(t)}")
        e("s_nop 1")
        e(f"v_permlane32_swap_b32 {vr(t)}, {vr(t + 1)}")
        e("s_nop 1")
        e(f"v_max_f32 {vr(t)}, {vr(t)}, {vr(t + 1)}")
        e(f"v_max_f32 {vr(t + 2)}, {vr(V_M + qb)}, {vr(t)}")                    # m_new
        e(f"v_cmp_neq_f32_e32 vcc, 0xff800000, {vr(t + 2)}")
        e(f"v_cndmask_b32_e32 {vr(t + 3)}, 0, {vr(t + 2)}, vcc")                # m_use: 0 while everything is masked
        al = V_E + 6 + qb                                                       # alpha of this row block (kept for O)
        e(f"v_cmp_neq_f32_e32 vcc, 0xff800000, {vr(V_M + qb)}")                 # rows that have seen a key before: only their O needs rescaling
        e(f"s_mov_b64 s[{S_TMP + 2 * qb}:{S_TMP + 2 * qb + 1}], vcc")
        e(f"v_sub_f32 {vr(al)}, {vr(V_M + qb)}, {vr(t + 3)}")
        e(f"v_exp_f32_e32 {vr(al)}, {vr(al)}")
        e(f"v_mov_b32 {vr(V_M + qb)}, {vr(t + 2)}")
        e(f"v_mov_b32 {vr(t + 4)}, 0")
        e(f"v_mul_f32 {vr(V_L + qb)}, {vr(V_L + qb)}, {vr(al)}")
        for jj in range(8):
            r = 2 * jj
            pw = p_word(qb, 1 if jj >= 4 else 0, jj % 4)
            rw = r_word(qb, 1 if jj >= 4 else 0, jj % 4)
            e0, e1, f0, f1 = V_E, V_E + 1, V_E + 2, V_E + 3
            e(f"v_sub_f32 {vr(e0)}, {sr[r]}, {vr(t + 3)}")
            e(f"v_sub_f32 {vr(e1)}, {sr[r + 1]}, {vr(t + 3)}")
            e(f"v_exp_f32_e32 {vr(e0)}, {vr(e0)}")
            e(f"v_exp_f32_e32 {vr(e1)}, {vr(e1)}")
            e("s_nop 0")
            e(f"{cvt} {vr(pw)}, {vr(e0)}, {vr(e1)}")
            e(f"v_add_f32 {vr(t + 4)}, {vr(t + 4)}, {vr(e0)}")
            e(f"v_add_f32 {vr(t + 4)}, {vr(t + 4)}, {vr(e1)}")
            if dtype == "bf16":
                e(f"v_lshlrev_b32_e32 {vr(f0)}, 16, {vr(pw)}")
                e(f"v_and_b32_e32 {vr(f1)}, 0xffff0000, {vr(pw)}")
            else:
                e(f"v_cvt_f32_f16_e32 {vr(f0)}, {vr(pw)}")
                e(f"v_cvt_f32_f16_sdwa {vr(f1)}, {vr(pw)} dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_1")
            e(f"v_sub_f32 {vr(e0)}, {vr(e0)}, {vr(f0)}")      # rounding residue of P, for the compensating product
            e(f"v_sub_f32 {vr(e1)}, {vr(e1)}, {vr(f1)}")
            e(f"{cvt} {vr(rw)}, {vr(e0)}, {vr(e1)}")
        e(f"v_add_f32 {vr(V_L + qb)}, {vr(V_L + qb)}, {vr(t + 4)}")
    # ---- rescale O where the reference of a row that already holds something moved (a row without keys so far holds
    # zeros whatever its alpha: the first half of a tree block skips the whole pass)
    e(f"v_cmp_neq_f32_e32 vcc, 1.0, {vr(V_E + 6)}")
    e(f"s_and_b64 s[{S_TMP + 4}:{S_TMP + 5}], vcc, s[{S_TMP}:{S_TMP + 1}]")
    e(f"v_cmp_neq_f32_e32 vcc, 1.0, {vr(V_E + 7)}")
    e(f"s_and_b64 vcc, vcc, s[{S_TMP + 2}:{S_TMP + 3}]")
    e(f"s_or_b64 vcc, vcc, s[{S_TMP + 4}:{S_TMP + 5}]")
    e("s_cbranch_vccz .Lnoscale_%=")
    for qb in range(2):
        for db in range(DB):
            base = A_O + 16 * (db * 2 + qb)
            for r in range(16):
                e(f"v_accvgpr_read_b32 {vr(t + 5)}, {ar(base + r)}")
                e(f"v_mul_f32 {vr(t + 5)}, {vr(t + 5)}, {vr(V_E + 6 + qb)}")
                e(f"v_accvgpr_write_b32 {ar(base + r)}, {vr(t + 5)}")
    e("s_nop 7")
    e(".Lnoscale_%=:")
    # ---- O += V^T P^T, and the same product with the residue of P
    for g in range(NV):
        e(f"s_waitcnt lgkmcnt({2 * min(PF - 1, NV - 1 - g)})")
        a = vr(V_VF + 4 * (g % PF), 4)
        for qb in range(2):
            cd = ar(A_O + 16 * ((g % DB) * 2 + qb), 16)
            e(f"{mfma} {cd}, {a}, {vr(p_word(qb, g // DB, 0), 4)}, {cd}")
        for qb in range(2):
            cd = ar(A_O + 16 * ((g % DB) * 2 + qb), 16)
            e(f"{mfma} {cd}, {a}, {vr(r_word(qb, g // DB, 0), 4)}, {cd}")
        if g + PF < NV:
            issue_v(g + PF)
    e("s_nop 15")   # the compiler does not know that MFMAs came last
    e("s_nop 15")
    return out


def operands_masked(D: int) -> str:
    KS, DB = D // 16, D // 32
    outs, ins = [], []
    for i in range(32 * DB):
        outs.append(f'"+{{a{A_O + i}}}"(w_o[{i}])')
    for i in range(2):
        outs.append(f'"+{{v{V_M + i}}}"(w_m[{i}])')
    for i in range(2):
        outs.append(f'"+{{v{V_L + i}}}"(w_l[{i}])')
    for i in range(8 * KS):
        ins.append(f'"{{a{A_Q + i}}}"(w_q[{i}])')
    for i in range(32):
        ins.append(f'"{{v{V_MADD + i}}}"(w_madd[{i}])')
    ins += [f'"{{v{V_KRD}}}"(w_krd)', f'"{{v{V_VRD}}}"(w_vrd)', f'"{{s{S_KCUR}}}"(w_koffs)', f'"{{s{S_VCUR}}}"(w_voffs)', f'"{{s{S_C}}}"(w_c)']
    clob = [f'"v{r}"' for r in list(range(V_R, V_R + 16)) + list(range(V_S, V_VF + 4 * PF)) + list(range(V_PS, V_T + 6))]
    clob += [f'"s{r}"' for r in range(S_TMP, S_TMP + 8)] + ['"vcc"', '"scc"', '"memory"']
    return "      : " + ", ".join(outs) + "\n      : " + ", ".join(ins) + "\n      : " + ", ".join(clob)



def _f32(x: float) -> str:
    import struct
    return struct.pack(">f", x).hex()


def operands(D: int) -> str:
    """The operand lists of the asm statement: every value in the register the code above names.
    Every operand is one 32-bit register. (Operands that are whole register tuples make the
    compiler copy tuples into and out of fixed registers around the statement, and hipcc's
    lowering of such copies between accumulation-register tuples is not reliable: it has
    produced wrong results and, in one configuration, an internal error.)
    C++ side names: float w_o[32 * DB], w_m[2], w_l[2]; uint32_t w_q[8 * KS]; scalars as declared in the
    kernel."""
    KS, DB = D // 16, D // 32
    outs, ins = [], []
    for i in range(32 * DB):
        outs.append(f'"+{{a{A_O + i}}}"(w_o[{i}])')
    for i in range(2):
        outs.append(f'"+{{v{V_M + i}}}"(w_m[{i}])')
    for i in range(2):
        outs.append(f'"+{{v{V_L + i}}}"(w_l[{i}])')
    outs += [f'"+{{s{S_KRUN}}}"(w_krun_lo)', f'"+{{s{S_KRUN + 1}}}"(w_krun_hi)', f'"+{{s{S_VRUN}}}"(w_vrun_lo)', f'"+{{s{S_VRUN + 1}}}"(w_vrun_hi)',
             f'"+{{s{S_KCUR}}}"(w_kcur)', f'"+{{s{S_KNEXT}}}"(w_knext)', f'"+{{s{S_VPREV}}}"(w_vprev)', f'"+{{s{S_VCUR}}}"(w_vcur)',
             f'"+{{s{S_PVOFF}}}"(w_pvoff)', f'"+{{s{S_NT}}}"(w_nt)', f'"+{{s{S_NREAL}}}"(w_nreal)']
    for i in range(8 * KS):
        ins.append(f'"{{a{A_Q + i}}}"(w_q[{i}])')
    ins += [f'"{{v{V_KRD}}}"(w_krd)', f'"{{v{V_VRD}}}"(w_vrd)', f'"{{v{V_KOFF}}}"(w_koff)', f'"{{v{V_VOFF}}}"(w_voff)',
            f'"{{s{S_KSTEP}}}"(w_kstep_lo)', f'"{{s{S_KSTEP + 1}}}"(w_kstep_hi)', f'"{{s{S_VSTEP}}}"(w_vstep_lo)', f'"{{s{S_VSTEP + 1}}}"(w_vstep_hi)',
            f'"{{s{S_KTILE}}}"(w_ktile_lo)', f'"{{s{S_KTILE + 1}}}"(w_ktile_hi)', f'"{{s{S_VTILE}}}"(w_vtile_lo)', f'"{{s{S_VTILE + 1}}}"(w_vtile_hi)',
            f'"{{s{S_KDST}}}"(w_kdst)', f'"{{s{S_VDST}}}"(w_vdst)', f'"{{s{S_C}}}"(w_c)']
    clob = [f'"v{r}"' for r in list(range(V_S, V_VF + 4 * PF)) + list(range(V_PS, V_T + 6))]
    # m0: the tile requests set it (the LDS destination of global_load_lds); the compiler's own requests around the
    # statement use it too and must not assume a value across it
    clob += [f'"s{r}"' for r in range(S_TMP, S_TMP + 8)] + ['"m0"', '"vcc"', '"scc"', '"memory"']
    return "      : " + ", ".join(outs) + "\n      : " + ", ".join(ins) + "\n      : " + ", ".join(clob)


# scalar instructions that leave a result in SCC
_SCC_WRITERS = ("s_add", "s_sub", "s_and_b", "s_or_b", "s_xor", "s_nand", "s_nor", "s_xnor", "s_lshl", "s_lshr", "s_ashr", "s_andn2", "s_orn2",
                "s_min", "s_max", "s_abs", "s_bfe", "s_not", "s_bcnt")


def verify(body: list[str], ops: str, name: str) -> None:
    """Raises if the assembly text touches a register the operand lists do not name. The compiler
    keeps its own values (addresses among them) in every register the statement does not
    declare, so an undeclared write is a wild pointer waiting to happen; an undeclared read is a
    value nobody set. The named registers (m0, vcc, scc, exec) are held to the same rule as the numbered ones: an
    instruction that writes one, openly or by its definition (compares, scalar arithmetic), needs it among the
    clobbers. Also checks that register tuples start on an even register."""
    import re
    decl = {"v": set(), "s": set(), "a": set()}
    inputs = {"v": set(), "s": set(), "a": set()}
    for m in re.finditer(r'"(\+?)\{([vas])(\d+)\}"', ops):
        (decl if m.group(1) else inputs)[m.group(2)].add(int(m.group(3)))
    for m in re.finditer(r'"([vs])(\d+)"', ops.split("\n")[-1]):
        decl[m.group(1)].add(int(m.group(2)))
    named_decl = set(re.findall(r'"(m0|vcc|scc|exec)"', ops.split("\n")[-1]))

    def named_writes(op, arglist):
        out = set()
        if not op.startswith(("s_cbranch", "s_branch", "s_waitcnt", "s_nop", "s_barrier", "global_load_lds", "s_cmp")) and arglist:
            head = arglist[0].split("_")[0]          # vcc_lo / exec_hi name a half of the pair
            if head in ("m0", "vcc", "exec"):
                out.add(head)
        if op.startswith("v_cmp") and op.endswith("_e32"):
            out.add("vcc")                           # the e32 form has no other destination
        if op.startswith("v_cmpx"):
            out.add("exec")
        if op.startswith(("s_cmp", "s_bitcmp")) or op.startswith(_SCC_WRITERS):
            out.add("scc")
        if "saveexec" in op or op.startswith("s_wrexec"):
            out.add("exec")
        return out

    def regs(tok):
        for m in re.finditer(r"\b([vas])\[(\d+):(\d+)\]|\b([vas])(\d+)\b", tok):
            if m.group(1):
                if m.group(1) != "s" and int(m.group(2)) % 2:
                    raise AssertionError(f"{name}: misaligned register tuple in `{tok}`")
                yield m.group(1), range(int(m.group(2)), int(m.group(3)) + 1)
            else:
                yield m.group(4), range(int(m.group(5)), int(m.group(5)) + 1)

    no_dst = ("s_cmp", "s_cbranch", "s_branch", "s_waitcnt", "s_nop", "s_barrier", "global_load_lds", "v_cmp")
    for line in body:
        line = line.split(";")[0].strip()
        if not line or line.endswith(":"):
            continue
        parts = line.split(None, 1)
        if len(parts) < 2:
            continue
        op, args = parts
        arglist = [a.strip() for a in args.split(",")]
        if op.startswith(no_dst):
            dst, src = [], (arglist[1:] if op.startswith("v_cmp") else arglist)
        else:
            dst, src = [arglist[0]], arglist[1:]
            if op.startswith(("v_dot2c", "v_permlane32_swap")):
                src = arglist
            if op.startswith("v_permlane32_swap"):
                dst = arglist
        for d in dst:
            for k, r in regs(d):
                bad = set(r) - decl[k]
                if bad:
                    raise AssertionError(f"{name}: `{line}` writes undeclared {k}{sorted(bad)}")
        bad_named = named_writes(op, arglist) - named_decl
        if bad_named:
            raise AssertionError(f"{name}: `{line}` writes undeclared {sorted(bad_named)}")
        for t in src:
            for k, r in regs(t):
                bad = set(r) - decl[k] - inputs[k]
                if bad:
                    raise AssertionError(f"{name}: `{line}` reads undeclared {k}{sorted(bad)}")


def hazards(body: list[str], name: str) -> None:
    """Raises if the text breaks one of the issue rules the hardware does not enforce itself (the assembler inserts
    nothing, and each of these showed up as wrong numbers on the GPU, never as a fault). Distances are in wait
    states: every instruction counts one, `s_nop n` counts n + 1. Checked in layout order.
      * the result of `v_dot2c` read by a different vector instruction: 3 wait states;
      * the result of a transcendental (`v_exp_f32`) read by a vector instruction: 1;
      * a write of M0 before the `global_load_lds` that uses it: 1;
      * a VGPR result of an 8-pass MFMA touched by a non-MFMA instruction: 11;
      * SCC: an `s_cselect` / `s_cbranch_scc` takes the compare before it, so nothing that writes SCC (`s_add`,
        `s_addc`, ...) may stand between them; an `s_addc` takes the carry of the `s_add_u32` before it;
      * the statement ends on at least 11 wait states without an MFMA (the compiler reads the accumulators next and
        does not know the statement holds MFMAs)."""
    import re
    reg = re.compile(r"\b([vas])(\d+)\b|\b([vas])\[(\d+):(\d+)\]")

    def regs(tok):
        out = set()
        for m in reg.finditer(tok):
            if m.group(1):
                out.add((m.group(1), int(m.group(2))))
            else:
                out.update((m.group(3), i) for i in range(int(m.group(4)), int(m.group(5)) + 1))
        return out

    ins = []
    for line in body:
        line = line.split(";")[0].strip()
        if not line or line.endswith(":"):
            continue
        parts = line.split(None, 1)
        ins.append((parts[0], [a.strip() for a in parts[1].split(",")] if len(parts) > 1 else [], line))

    def dst_src(op, args):
        every = set().union(*[regs(a) for a in args]) if args else set()
        if op.startswith(("s_cmp", "s_cbranch", "s_branch", "s_waitcnt", "s_nop", "s_barrier", "global_load_lds")):
            return set(), every
        if op.startswith("v_cmp"):
            return set(), set().union(*[regs(a) for a in args[1:]])
        d = regs(args[0]) if args else set()
        src = set().union(*[regs(a) for a in args[1:]]) if len(args) > 1 else set()
        if op.startswith(("v_dot2c", "v_permlane32_swap")):
            src |= d
        if op.startswith("v_permlane32_swap"):
            d |= regs(args[1])
        return d, src

    def wait_states(op, args):
        return int(args[0]) + 1 if op == "s_nop" else 1

    def too_close(i, need, offends):
        dist = 0
        for j in range(i + 1, len(ins)):
            op, args, text = ins[j]
            if offends(op, args):
                raise AssertionError(f"{name}: `{text}` follows `{ins[i][2]}` after {dist} wait states, needs {need}")
            dist += wait_states(op, args)
            if dist >= need:
                return

    scc_writers = _SCC_WRITERS
    for i, (op, args, text) in enumerate(ins):
        d, _ = dst_src(op, args)
        if op.startswith("v_dot2c"):
            too_close(i, 3, lambda o, a: o.startswith("v_") and not o.startswith("v_dot2c") and dst_src(o, a)[1] & d)
        if op.startswith(("v_exp_f32", "v_log_f32", "v_rcp_f32", "v_rsq_f32", "v_sqrt_f32")):
            too_close(i, 1, lambda o, a: o.startswith("v_") and dst_src(o, a)[1] & d)
        if op == "s_mov_b32" and args[0] == "m0":
            too_close(i, 1, lambda o, a: o.startswith("global_load_lds"))
        if op.startswith("v_mfma"):
            vd = {r for r in d if r[0] == "v"}
            if vd:
                too_close(i, 11, lambda o, a: not o.startswith(("v_mfma", "s_")) and (dst_src(o, a)[0] | dst_src(o, a)[1]) & vd)
        if op.startswith(("s_cselect", "s_cbranch_scc", "s_addc")):
            for j in range(i - 1, -1, -1):
                o = ins[j][0]
                if o.startswith("s_cmp"):
                    if op.startswith("s_addc"):
                        raise AssertionError(f"{name}: `{text}` takes its carry from `{ins[j][2]}`")
                    break
                if o.startswith(scc_writers):
                    if not (op.startswith("s_addc") and o.startswith("s_add_u32")):
                        raise AssertionError(f"{name}: `{ins[j][2]}` overwrites SCC before `{text}`")
                    break
            else:
                raise AssertionError(f"{name}: nothing sets SCC before `{text}`")
    tail = 0
    for op, args, text in reversed(ins):
        if op.startswith("v_mfma") or op.startswith(("s_branch", "s_cbranch")):
            break
        tail += wait_states(op, args)
    if tail < 11:
        raise AssertionError(f"{name}: the statement ends {tail} wait states after an MFMA or a branch, needs 11")


def render() -> str:
    lines = ["// Generated by gen_wide_loop.py - do not edit; edit the generator and run it.", "// clang-format off",
             "#ifndef FTA_WIDE_LOOP_ASM_INC", "#define FTA_WIDE_LOOP_ASM_INC"]
    for D in (128, 64):
        L = layout(D)
        for dtype in ("bf16", "f16"):
            body = gen(D, dtype)
            verify(body, operands(D), f"loop {D} {dtype}")
            hazards(body, f"loop {D} {dtype}")
            lines.append(f"#define FTA_WIDE_LOOP_{D}_{dtype.upper()}() asm volatile( \\")
            for ins in body:
                lines.append(f'      "{ins}\\n\\t" \\')
            lines.append(operands(D).replace("\n", " \\\n") + ")")
            for H in (0, 1):
                lines.append(f"#define FTA_WIDE_MASKED_{D}_{dtype.upper()}_H{H}() asm volatile( \\")
                mbody = gen_masked(D, dtype, H)
                verify(mbody, operands_masked(D), f"masked {D} {dtype} H{H}")
                hazards(mbody, f"masked {D} {dtype} H{H}")
                for ins in mbody:
                    lines.append(f'      "{ins}\\n\\t" \\')
                lines.append(operands_masked(D).replace("\n", " \\\n") + ")")
        lines.append(f"static_assert(fta::TileLayout<{D}>::kTileBytes == {L['tile']} && fta::TileLayout<{D}>::kBlockPitch == {L['pitch']} && "
                     f"fta::TileLayout<{D}>::kChunkStride == {L['chunk']} && fta::TileLayout<{D}>::kRowsPerBlock == {L['rpb']}, "
                     f"\"gen_wide_loop.py and TileLayout<{D}> disagree\");")
    lines.append("#endif  // FTA_WIDE_LOOP_ASM_INC")
    lines.append("// clang-format on")
    return "\n".join(lines) + "\n"


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "wide_loop_asm.inc")
    with open(path, "w") as f:
        f.write(render())
    print(f"wrote {path}")
