#!/usr/bin/env python3
"""Writes sdpa_prefill_hot.inc: the instruction streams of the steady-state iteration of the
64-rows-per-wavefront prefill kernel (sdpa_prefill_mfma64.hip), one per LDS ring slot and storage type.

Why generated text and not compiler output: in that kernel a wavefront owns a SIMD alone, so each of its
instructions costs one of the eight issue slots an MFMA lasts; the loop only pays off when every slot is
planned (two exponentials and a pack, or two reductions, plus one LDS read under each MFMA; no register
copies).  The register assignment below is fixed and shared with the kernel source through the
PF_R_* macros it also emits.

    python3 gen_prefill_hot.py > sdpa_prefill_hot.inc
"""

D = 128
ROWB = D * 2            # bytes of one K/V row in LDS
TN = 32                 # keys per tile
TILE = TN * ROWB        # 8 KiB
RING = 8                # K tiles and V tiles resident in LDS (the loop below is unrolled once per slot)
NSTEP = D // 16         # 8 k-steps of the score product
NDB = D // 32           # 4 blocks of the head dimension
QB = 2                  # 32-row query blocks per wavefront

# ---- VGPR map ---------------------------------------------------------------------------------------------
S = [[0, 16], [32, 48]]          # S[par][qb]: first register of a 16-register score tuple
NR = [64, 80]                    # -m_ref splat per query block (initial accumulator of the score product)
P = 96                           # 16 packed probability dwords: pair p = qb*8 + ks*4 + j at P + p
KB = 112                         # K operands of one tile: k-step s at KB + 4*s
VB = 144                         # V operands of one tile: operand i = ks*NDB + db at VB + 4*i
KADDR = 176                      # 8 LDS byte offsets (inside a tile) of the K operand of k-step s
VADDR = 184                      # 8 LDS byte addresses of the V operand halves in ring slot 0 (V ring base included): VADDR + 2*db + h
E = 192                          # 4 temporaries for exponentials
MX = [196, 197]                  # running maxima of the next score tile per query block (this lane's keys)
LRUN = [198, 199]                # row sums (this lane's keys)
KVOFF = [200, 201]               # byte offsets of this lane's two 16-byte pieces of a K tile in global memory
VVOFF = [202, 203]               # same for a V tile
REL = [204, 205]                 # masked loop: this lane's key limit minus the first key it holds of the NEXT tile, per query block
NEGINF = 206                     # -inf
THR = [207, 208]                 # per query: 8.0 once its reference maximum is set, -inf before (the tile maximum is compared to it)
MREF = [209, 210]                # reference maxima (log2 units)
TT = [211, 212, 213, 214]        # temporaries of the rescaling code
# ---- SGPR map (all pinned by the asm statement's operand list) ------------------------------------------------
KDESC = 40                       # s[40:43] buffer descriptor of the next K tile to load (base, base_hi, bytes, flags)
VDESC = 44                       # s[44:47] same for V
KSTEP, VSTEP = 48, 49            # bytes from one tile to the next
T, LEFT = 50, 52                 # pending tile index (in/out), tiles left to process (in/out)
TMP = 59
NHOT = 60                        # tiles below this index need no mask
SC0, SC1 = 62, 64                # s[62:63], s[64:65]: lane masks in the rescaling code
LDSW = 53                        # LDS byte address of this wavefront's first 1 KiB piece of K ring slot 0
M0SAVE = 56
KREM, VREM = 57, 58              # signed bytes from the next tile's first row to the end of the tensor slice
DRAWADDR = 66                    # s[66:67] address of the work counter this workgroup draws its items from
DRAWAT = 68                      # draw the next item when this many tiles are left (never reached: no draw from this wavefront)
DRAWN, DRAWONE = 192, 193        # AGPRs: the counter's answer (lane 0) and the constant 1 it is advanced by
# ---- AGPR map ---------------------------------------------------------------------------------------------
def O(db, qb):                   # O^T accumulators
    return (db * QB + qb) * 16
def Q(qb, s):                    # Q^T operands
    return 128 + (qb * NSTEP + s) * 4


def v(a, n=1):
    return "v%d" % a if n == 1 else "v[%d:%d]" % (a, a + n - 1)


def a_(a, n):
    return "a[%d:%d]" % (a, a + n - 1)


def block(slot, ty):
    """One iteration u (u % RING == slot): scores of tile u+1 with the probabilities of tile u underneath, then
    O^T += V(u)^T P(u)^T with the row sums of P(u), the maxima of S(u+1) and the K operand reads of tile u+2.
    LDS reads are issued in the first half of each product so that they have landed when the next one starts."""
    mfma = "v_mfma_f32_32x32x16_%s" % ty
    pack = "v_cvt_pk_%s_f32" % ty
    dot2 = "v_dot2c_f32_%s" % ty
    ones = {"bf16": "0x3f803f80", "f16": "0x3c003c00"}[ty]
    par = slot % 2
    sc, sn = S[par], S[1 - par]
    L = []
    # K operands of tile u+1 were read during the previous iteration's second half
    L.append("s_waitcnt lgkmcnt(0)")
    for s in range(NSTEP):
        for qb in range(QB):
            m = s * QB + qb
            c = NR[qb] if s == 0 else sn[qb]
            L.append("%s %s, %s, %s, %s" % (mfma, v(sn[qb], 16), v(KB + 4 * s, 4), a_(Q(qb, s), 4), v(c, 16)))
            pi = m                                     # pair of score registers 2*(pi%8), +1 of query block pi/8
            src = sc[pi // 8] + 2 * (pi % 8)
            e = E + 2 * (m % 2)
            L.append("v_exp_f32 %s, %s" % (v(e), v(src)))
            L.append("v_exp_f32 %s, %s" % (v(e + 1), v(src + 1)))
            if m > 0:                                  # pack the previous pair: its exponentials have landed
                pe = E + 2 * ((m - 1) % 2)
                L.append("%s %s, %s, %s" % (pack, v(P + pi - 1), v(pe), v(pe + 1)))
            if m < 8:                                  # V operand m (both halves) for the product below
                i = m
                ks, db = i // NDB, i % NDB
                off = slot * TILE + ks * 16 * ROWB
                for h in range(2):
                    L.append("ds_read_b64_tr_b16 %s, %s offset:%d" % (v(VB + 4 * i + 2 * h, 2), v(VADDR + 2 * db + h), off))
    last = NSTEP * QB - 1
    pe = E + 2 * (last % 2)
    L.append("s_nop 0")
    L.append("%s %s, %s, %s" % (pack, v(P + last), v(pe), v(pe + 1)))
    L.append("s_add_i32 s%d, s%d, 1" % (TMP, T))
    L += mask_clump(sn, ".Lnomask%d_%%=" % slot)
    L.append("s_waitcnt lgkmcnt(0)")
    for i in range(2 * NDB):
        for qb in range(QB):
            m = i * QB + qb
            ks, db = i // NDB, i % NDB
            o = O(db, qb)
            L.append("%s %s, %s, %s, %s" % (mfma, a_(o, 16), v(VB + 4 * i, 4), v(P + qb * 8 + ks * 4, 4), a_(o, 16)))
            for j in range(2):
                if m < 8:                              # row sums of P(u): 16 pairs
                    p = 2 * m + j
                    L.append("%s %s, %s, %s" % (dot2, v(LRUN[p // 8]), ones, v(P + p)))
                else:                                  # maxima of S(u+1): 8 pairs per query block
                    x = 2 * (m - 8) + j
                    q2, e8 = x // 8, x % 8
                    r0 = sn[q2] + 2 * e8
                    if e8 == 0:
                        L.append("v_max_f32 %s, %s, %s" % (v(MX[q2]), v(r0), v(r0 + 1)))
                    else:
                        L.append("v_max3_f32 %s, %s, %s, %s" % (v(MX[q2]), v(MX[q2]), v(r0), v(r0 + 1)))
            if m < 8:                                  # K operand of k-step m of tile u+2 (its slot was read by the scores above)
                off = ((slot + 2) % RING) * TILE
                L.append("ds_read_b128 %s, %s offset:%d" % (v(KB + 4 * m, 4), v(KADDR + m), off))
    return L


def load_tile(desc, step, rem, voff, lds_off):
    """Start the global->LDS copy of the tile the descriptor points at and advance the descriptor.  Past the end of
    the tensor the remaining size is clamped to 0: the load then touches no memory (and its LDS slot is never read)."""
    L = []
    L.append("s_max_i32 s%d, s%d, 0" % (desc + 2, rem))
    L.append("s_add_u32 m0, s%d, %d" % (LDSW, lds_off))
    L.append("s_nop 0")
    L.append("buffer_load_dwordx4 %s, s[%d:%d], 0 offen lds" % (v(voff[0]), desc, desc + 3))
    L.append("s_add_u32 m0, m0, 0x400")
    L.append("s_nop 0")
    L.append("buffer_load_dwordx4 %s, s[%d:%d], 0 offen lds" % (v(voff[1]), desc, desc + 3))
    L.append("s_add_u32 s%d, s%d, s%d" % (desc, desc, step))
    L.append("s_addc_u32 s%d, s%d, 0" % (desc + 1, desc + 1))
    L.append("s_sub_i32 s%d, s%d, s%d" % (rem, rem, step))
    return L


def turn(slot):
    """Before tile t (t % RING == slot, slot even): the copies started three turns ago are complete for everyone (each
    turn starts exactly 8 per wavefront, so at most 16 may still be in flight); then K(t+8), K(t+9), V(t+6), V(t+7)
    start into the ring slots consumed since."""
    L = ["s_waitcnt vmcnt(16) lgkmcnt(0)", "s_barrier"]
    L += load_tile(KDESC, KSTEP, KREM, KVOFF, ((slot + 0) % RING) * TILE)
    L += load_tile(KDESC, KSTEP, KREM, KVOFF, ((slot + 1) % RING) * TILE)
    L += load_tile(VDESC, VSTEP, VREM, VVOFF, (RING + (slot + 6) % RING) * TILE)
    L += load_tile(VDESC, VSTEP, VREM, VVOFF, (RING + (slot + 7) % RING) * TILE)
    return L


def mask_clump(sn, label):
    """Mask the score tile in `sn` (two 16-register tuples) against REL when its index (in TMP) is not below N_HOT:
    register r of a score block is key 8*(r/4) + (r%4) (+ 4*g, already in REL), masked when that is >= REL.  Rare
    (a wavefront's last tiles), so one clump, skipped by a scalar branch.  Always moves REL on to the next tile."""
    L = ["s_cmp_lt_i32 s%d, s%d" % (TMP, NHOT), "s_cbranch_scc1 %s" % label]
    L += ["s_nop 7", "s_nop 7"]                        # the scores come out of the matrix pipe
    for q2 in range(QB):
        for r in range(16):
            kofs = 8 * (r // 4) + (r % 4)
            L.append("v_cmp_ge_i32 vcc, %d, %s" % (kofs, v(REL[q2])))
            L.append("v_cndmask_b32 %s, %s, %s, vcc" % (v(sn[q2] + r), v(sn[q2] + r), v(NEGINF)))
    L.append(label + ":")
    for q2 in range(QB):
        L.append("v_subrev_u32 %s, %d, %s" % (v(REL[q2]), TN, v(REL[q2])))
    return L


def check(par):
    """The pending tile (parity par) has a maximum above what its reference allows (2^8 above it, or any finite
    value while the reference is not set yet): go and move the reference."""
    return ["v_cmp_lt_f32 vcc, %s, %s" % (v(THR[0]), v(MX[0])),
            "v_cmp_lt_f32 s[%d:%d], %s, %s" % (SC0, SC0 + 1, v(THR[1]), v(MX[1])),
            "s_or_b64 vcc, vcc, s[%d:%d]" % (SC0, SC0 + 1),
            "s_cbranch_vccnz .Lresc%d_%%=" % par]


def resume():
    """Continue with tile T: leave if nothing is left, else go to the code in front of its ring slot's block."""
    L = ["s_cmp_eq_u32 s%d, 0" % LEFT, "s_cbranch_scc1 .Lexit_%=", "s_and_b32 s%d, s%d, %d" % (TMP, T, RING - 1)]
    for slot in range(1, RING):
        L += ["s_cmp_eq_u32 s%d, %d" % (TMP, slot), "s_cbranch_scc1 .Lpre%d_%%=" % slot]
    L += ["s_branch .Lpre0_%="]
    return L


def rescale(par):
    """Move the reference maxima of the pending tile (scores in S[par]) where its maximum asks for it; rescale the
    accumulators, the row sums and the pending scores.  Lanes that do not need it move by 0 (factor 1)."""
    L = [".Lresc%d_%%=:" % par, "s_nop 15"]             # O^T was written by the last MFMAs
    t0, t1, dl, al = TT
    for qb in range(QB):
        # tile maximum over both halves of the query's lanes
        L += ["v_mov_b32 %s, %s" % (v(t0), v(MX[qb])), "v_mov_b32 %s, %s" % (v(t1), v(MX[qb])),
              "s_nop 1", "v_permlane32_swap_b32 %s, %s" % (v(t0), v(t1)), "s_nop 1",
              "v_max_f32 %s, %s, %s" % (v(t0), v(t0), v(t1))]
        # need = tmax > THR; inited = THR > 0
        L += ["v_cmp_lt_f32 vcc, %s, %s" % (v(THR[qb]), v(t0)),
              "v_cmp_lt_f32 s[%d:%d], 0, %s" % (SC1, SC1 + 1, v(THR[qb])),
              "v_cndmask_b32 %s, 0, %s, vcc" % (v(dl), v(t0)),                                # delta
              "v_exp_f32_e64 %s, -%s" % (v(al), v(dl)),
              "v_mov_b32 %s, 0x41000000" % v(t1),
              "v_cndmask_b32 %s, %s, %s, vcc" % (v(THR[qb]), v(THR[qb]), v(t1)),              # reference set from now on
              "v_cndmask_b32_e64 %s, 1.0, %s, s[%d:%d]" % (v(al), v(al), SC1, SC1 + 1),       # nothing accumulated yet: factor 1
              "v_add_f32 %s, %s, %s" % (v(MREF[qb]), v(MREF[qb]), v(dl)),
              "v_mul_f32 %s, %s, %s" % (v(LRUN[qb]), v(LRUN[qb]), v(al))]
        for r in range(16):
            L.append("v_sub_f32 %s, 0, %s" % (v(NR[qb] + r), v(MREF[qb])))
        for r in range(16):
            L.append("v_sub_f32 %s, %s, %s" % (v(S[par][qb] + r), v(S[par][qb] + r), v(dl)))
        for db in range(NDB):
            for r in range(16):
                L += ["v_accvgpr_read_b32 %s, a%d" % (v(t0), O(db, qb) + r),
                      "v_mul_f32 %s, %s, %s" % (v(t0), v(t0), v(al)),
                      "v_accvgpr_write_b32 a%d, %s" % (O(db, qb) + r, v(t0))]
    L += ["s_nop 7"]
    L += resume()
    return L


def prologue():
    """State of a new work item: the K operands of tile 0 on their way from LDS, Q^T moved from the registers it
    arrives in (the score registers, free until the first product) to its AGPRs, O^T, row sums, reference maxima
    zero, no reference maximum set."""
    L = []
    for s_ in range(NSTEP):
        L.append("ds_read_b128 %s, %s" % (v(KB + 4 * s_, 4), v(KADDR + s_)))
    for i in range(QB * NSTEP * 4):
        L.append("v_accvgpr_write_b32 a%d, v%d" % (Q(0, 0) + i, i))
    for i in range(NDB * QB * 16):
        L.append("v_accvgpr_write_b32 a%d, 0" % i)
    for qb in range(QB):
        for i in range(16):
            L.append("v_mov_b32 %s, 0" % v(NR[qb] + i))
    for qb in range(QB):
        L.append("v_mov_b32 %s, %s" % (v(MX[qb]), v(NEGINF)))
        L.append("v_mov_b32 %s, %s" % (v(THR[qb]), v(NEGINF)))
        L.append("v_mov_b32 %s, 0" % v(MREF[qb]))
        L.append("v_mov_b32 %s, 0" % v(LRUN[qb]))
    return L


def first_scores(ty):
    """Scores of tile 0 from the K operands in KB (nothing to overlap with yet); K operands of tile 1 behind them."""
    mfma = "v_mfma_f32_32x32x16_%s" % ty
    sn = S[0]
    L = ["s_waitcnt lgkmcnt(0)"]
    for s_ in range(NSTEP):
        for qb in range(QB):
            c = NR[qb] if s_ == 0 else sn[qb]
            L.append("%s %s, %s, %s, %s" % (mfma, v(sn[qb], 16), v(KB + 4 * s_, 4), a_(Q(qb, s_), 4), v(c, 16)))
        L.append("ds_read_b128 %s, %s offset:%d" % (v(KB + 4 * s_, 4), v(KADDR + s_), 1 * TILE))
    L += ["s_mov_b32 s%d, 0" % TMP]
    L += mask_clump(sn, ".Lnomask_first_%=")
    L += ["s_nop 7", "s_nop 7"]
    for qb in range(QB):
        L.append("v_max_f32 %s, %s, %s" % (v(MX[qb]), v(sn[qb]), v(sn[qb] + 1)))
        for e8 in range(1, 8):
            L.append("v_max3_f32 %s, %s, %s, %s" % (v(MX[qb]), v(MX[qb]), v(sn[qb] + 2 * e8), v(sn[qb] + 2 * e8 + 1)))
    return L


def draw(slot):
    """Out of line, once per work item and workgroup: lane 0 advances the work counter.  The answer is not waited
    for here; it is one more (older) entry in the queue the turns count, which only makes their wait safer."""
    return [".Ldraw%d_%%=:" % slot,
            "s_mov_b64 s[%d:%d], exec" % (SC0, SC0 + 1),
            "s_mov_b64 exec, 1",
            "v_mov_b32 %s, 0" % v(E),
            "global_atomic_add a%d, %s, a%d, s[%d:%d] sc0" % (DRAWN, v(E), DRAWONE, DRAWADDR, DRAWADDR + 1),
            "s_mov_b64 exec, s[%d:%d]" % (SC0, SC0 + 1),
            "s_branch .Ldrawn%d_%%=" % slot]


def loop(ty):
    """The whole main path of a wavefront: tiles 0 .. LEFT-1.  Entry: T = 0, Q^T (scaled) in v0..v63, REL for tile 0,
    the copies of K(0..7), V(0..5) started (K(0..3), V(0), V(1) complete and visible).  Exit: T = LEFT tiles done (if
    T is even its turn has NOT been taken), O^T in its AGPRs, the row sums in LRUN, the reference maxima in MREF."""
    L = ["s_mov_b32 s%d, m0" % M0SAVE]
    L += prologue()
    L += first_scores(ty)
    L += ["s_branch .Lresc0_%="]                        # the first reference maximum
    for slot in range(RING):
        if slot > 0 and slot % 2 == 0:
            L += [".Lpre%d_%%=:" % slot] + turn(slot)
        elif slot % 2 == 1:
            L += [".Lpre%d_%%=:" % slot]
        L += [".Lslot%d_%%=:" % slot]
        L += block(slot, ty) + ["s_add_i32 s%d, s%d, 1" % (T, T), "s_sub_i32 s%d, s%d, 1" % (LEFT, LEFT)]
        L += ["s_cmp_eq_u32 s%d, s%d" % (LEFT, DRAWAT), "s_cbranch_scc1 .Ldraw%d_%%=" % slot, ".Ldrawn%d_%%=:" % slot]
        L += check(1 - slot % 2)
        L += ["s_cmp_eq_u32 s%d, 0" % LEFT, "s_cbranch_scc1 .Lexit_%="]
    L += [".Lpre0_%=:"] + turn(0)
    L += ["s_branch .Lslot0_%="]
    L += rescale(0)
    L += rescale(1)
    for slot in range(RING):
        L += draw(slot)
    L += [".Lexit_%=:", "s_mov_b32 m0, s%d" % M0SAVE, "s_nop 15"]
    return L


def main():
    out = []
    out.append("// Generated by gen_prefill_hot.py - do not edit.  Register map of the steady-state iteration:")
    out.append("//   VGPR  S[par][qb] %s  -m_ref %s  P %d..%d  K operands %d..%d  V operands %d..%d" %
               (S, NR, P, P + 15, KB, KB + 31, VB, VB + 31))
    out.append("//         K read offsets %d..%d  V read offsets %d..%d  temporaries %d..%d  maxima %s  row sums %s" %
               (KADDR, KADDR + 7, VADDR, VADDR + 7, E, E + 3, MX, LRUN))
    out.append("//   AGPR  O^T[db][qb] at 16*(2*db+qb)  Q^T[qb][s] at 128 + 4*(8*qb+s)")
    for name, val in (("S00", S[0][0]), ("S01", S[0][1]), ("S10", S[1][0]), ("S11", S[1][1]), ("NR0", NR[0]), ("NR1", NR[1]),
                      ("KB", KB), ("KADDR", KADDR), ("VADDR", VADDR), ("MX0", MX[0]), ("MX1", MX[1]),
                      ("LRUN0", LRUN[0]), ("LRUN1", LRUN[1])):
        out.append("#define PF_R_%s %d" % (name, val))
    clob = (list(range(NR[0], NR[0] + 16)) + list(range(NR[1], NR[1] + 16)) + list(range(P, P + 16)) + list(range(KB, KB + 32)) +
            list(range(VB, VB + 32)) + list(range(E, E + 4)) + MX + THR + TT)
    aclob = list(range(Q(0, 0), Q(0, 0) + QB * NSTEP * 4))
    # operand lists of the asm statement; the kernel source declares variables with these names
    outs = []
    for qb in range(QB):
        for s_ in range(NSTEP):            # Q^T arrives in the score registers, which the loop then overwrites
            outs.append('"+{%s}"(qreg[%d][%d])' % (v((qb * NSTEP + s_) * 4, 4), qb, s_))
    for qb in range(QB):
        outs.append('"={%s}"(l_run[%d])' % (v(LRUN[qb]), qb))
    for qb in range(QB):
        outs.append('"={%s}"(m_ref[%d])' % (v(MREF[qb]), qb))
    for db in range(NDB):
        for qb in range(QB):
            outs.append('"={%s}"(o_acc[%d][%d])' % (a_(O(db, qb), 16), db, qb))
    ins = []
    for s_ in range(NSTEP):
        ins.append('"{%s}"(k_addr[%d])' % (v(KADDR + s_), s_))
    for db in range(NDB):
        for h in range(2):
            ins.append('"{%s}"(v_addr[%d][%d])' % (v(VADDR + 2 * db + h), db, h))
    for c in range(2):
        ins.append('"{%s}"(k_voff[%d])' % (v(KVOFF[c]), c))
    for c in range(2):
        ins.append('"{%s}"(v_voff[%d])' % (v(VVOFF[c]), c))
    for qb in range(QB):
        outs.append('"+{%s}"(hot_rel[%d])' % (v(REL[qb]), qb))
    ins.append('"{%s}"(hot_neg_inf)' % v(NEGINF))
    # scalar state of the loop
    outs.append('"+{s[%d:%d]}"(hot_kdesc)' % (KDESC, KDESC + 3))
    outs.append('"+{s[%d:%d]}"(hot_vdesc)' % (VDESC, VDESC + 3))
    outs.append('"+{s%d}"(hot_t)' % T)
    outs.append('"+{s%d}"(hot_left)' % LEFT)
    outs.append('"+{s%d}"(hot_krem)' % KREM)
    outs.append('"+{s%d}"(hot_vrem)' % VREM)
    ins.append('"{s%d}"(hot_kstep)' % KSTEP)
    ins.append('"{s%d}"(hot_vstep)' % VSTEP)
    ins.append('"{s%d}"(hot_ldsw)' % LDSW)
    ins.append('"{s%d}"(hot_nhot)' % NHOT)
    ins.append('"{s[%d:%d]}"(hot_drawaddr)' % (DRAWADDR, DRAWADDR + 1))
    ins.append('"{s%d}"(hot_drawat)' % DRAWAT)
    ins.append('"{a%d}"(hot_one)' % DRAWONE)
    outs.append('"+{a%d}"(drawn)' % DRAWN)
    clob_all = ['"v%d"' % r for r in clob] + ['"a%d"' % r for r in aclob] + ['"s%d"' % r for r in (M0SAVE, TMP, SC0, SC0 + 1, SC1, SC1 + 1)] + ['"vcc"', '"scc"', '"memory"']
    out.append("#define PF_HOT_OPERANDS \\")
    out.append("    : %s \\" % ", ".join(outs))
    out.append("    : %s \\" % ", ".join(ins))
    out.append("    : %s" % ", ".join(clob_all))
    for ty in ("bf16", "f16"):
        for once in (0,):
            lines = loop(ty)
            out.append("#define PF_HOT_%s \\" % ty.upper())
            for k, ln in enumerate(lines):
                end = "" if k == len(lines) - 1 else " \\"
                out.append('    "%s\\n\\t"%s' % (ln, end))
    print("\n".join(out))


if __name__ == "__main__":
    main()
