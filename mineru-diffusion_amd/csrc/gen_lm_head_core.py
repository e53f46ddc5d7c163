#!/usr/bin/env python3
"""Generator of lm_head_core.inc: the hand-scheduled gfx950 core of the fused vocabulary projection +
confidence reduction (logits = x . W^T never leave the chip; what leaves is one (max, sum of exp, first
argmax) record per x row and 128-column slice of the vocabulary).

Run  python gen_lm_head_core.py > lm_head_core.inc  after changing the schedule; the .inc file is what the
build compiles.

Work of one workgroup (4 wavefronts, one per SIMD): a tile of 256 vocabulary rows of W x 256 rows of x, the
whole hidden dimension.  A wavefront owns 128 vocabulary rows x 128 x rows = 4 x 4 MFMA tiles of 32 x 32,
i.e. all 256 accumulation registers:
    D[vocab, x row] += W fragment (A, 32 vocab rows x 16 k) . x fragment (B, 16 k x 32 x rows)
so that an x row lives in one lane (two lanes: the halves of the wavefront hold different vocab rows of it) and
the reduction over the vocabulary needs no cross-lane work until the very end.

LDS: two stages of 64 KB; a stage holds one k-block of 64 elements: W tile (256 rows x 128 bytes) then x tile
(same).  The 16-byte chunk c of row r sits at position c ^ ((r >> 1) & 7): ds_read_b128 of 16 consecutive rows
then covers all 64 banks once, and the address of k-step ks is that of k-step 0 XOR (ks << 5).  Tiles are
filled by global_load_lds_dwordx4 (1 KB = 8 rows per instruction, 16 instructions per wavefront and k-block).

Iteration kb (stage kb & 1), four k-steps of 16 MFMAs; fragments of k-step ks sit in ring half ks & 1:
  k-steps 0..2: MFMAs of the step || ds_reads of the next step's 8 fragments
  k-step 3:     wait for this wavefront's loads of k-block kb+1 and for its own reads of k-block kb; barrier
                (now k-block kb+1 is visible to all, and nobody reads stage kb & 1 any more: the fragments of
                k-step 3 are in registers); MFMAs || ds_reads of k-step 0 of k-block kb+1 from the other stage
                || the 16 loads of k-block kb+2 into this stage
One barrier per 64 MFMAs, the MFMA / fragment stream never drains.

Epilogue, per tile of 32 x rows: the lane's 64 logits (4 vocab tiles x 16 registers, ascending vocab index)
are rounded to bf16 (the projection's output type in the reference, embed_head.py:61-67) and reduced to
(max, first index of the max, sum of exp2((x - max) c)); the two half-wavefronts are merged and lanes 0..31
store one 16-byte record per x row.

Physical registers (all clobbered; the compiler keeps v0..v15 for operands):
  v16..v23 temporaries       v24..v31 W fragment addresses [stage][k-step]   v32..v39 x fragment addresses
  v40..v47 W load offsets    v48..v55 x load offsets                          v56..v63 epilogue state
  v64..v127 epilogue values  v128..v143 epilogue temporaries                  v192..v255 fragment ring (2 x 8 x 4)
  a0..a255 accumulators [vocab tile][x tile][16]                               s40..s59 loop state
"""
import sys

MFMA = "v_mfma_f32_32x32x16_bf16"
ROW = 128                          # bytes per LDS row (64 bf16)
TILE = 256 * ROW                   # 32768: one operand tile of a stage
STAGE = 2 * TILE
NDMA = 8                           # loads per operand, wavefront and k-block

T = [f"v{16 + i}" for i in range(8)]
AW = [[f"v{24 + 4 * s + ks}" for ks in range(4)] for s in range(2)]
AX = [[f"v{32 + 4 * s + ks}" for ks in range(4)] for s in range(2)]
GW = [f"v{40 + j}" for j in range(8)]
GX = [f"v{48 + j}" for j in range(8)]
NEG_INF, PO, XR, VL = "v56", "v57", "v58", "v59"
GT, DUMMY = "v60", "v61"                   # touch prefetch: this lane's row offset in W, and where the touched word lands
E = [f"v{64 + e}" for e in range(64)]
U = [f"v{128 + i}" for i in range(16)]

S_KB, S_TMP, S_DST0, S_DST1 = "s40", "s41", "s42", "s43"
S_WB, S_XB, S_SAVE = "s[44:45]", "s[46:47]", "s[48:49]"
S_WB_LO, S_WB_HI, S_XB_LO, S_XB_HI = "s44", "s45", "s46", "s47"
S_TB, S_TB_LO, S_TB_HI, S_TBLK, S_NKB1 = "s[50:51]", "s50", "s51", "s52", "s53"
TOUCH_AHEAD = 4                    # the loop touches k-block kb + 4 while it loads k-block kb + 2


def acc(vt, xt, i=None):
    r = (vt * 4 + xt) * 16
    return f"a[{r}:{r + 15}]" if i is None else f"a{r + i}"


def frag(half, slot):
    r = 192 + 32 * half + 4 * slot
    return f"v[{r}:{r + 3}]"


# fragment slots of a ring half: 0..3 = W fragments of vocab tiles 0..3, 4..7 = x fragments of x tiles 0..3
READ_ORDER = [0, 4, 5, 1, 6, 2, 7, 3]                      # A0 B0 B1 A1 B2 A2 B3 A3
MFMA_ORDER = [(0, 0), (0, 1), (1, 0), (1, 1), (0, 2), (1, 2), (2, 0), (2, 1), (2, 2),
              (0, 3), (1, 3), (2, 3), (3, 0), (3, 1), (3, 2), (3, 3)]


def read_op(stage, ks, half, slot):
    if slot < 4:
        off = 4096 * slot
        return f"ds_read_b128 {frag(half, slot)}, {AW[stage][ks]}" + (f" offset:{off}" if off else "")
    off = 4096 * (slot - 4)
    return f"ds_read_b128 {frag(half, slot)}, {AX[stage][ks]}" + (f" offset:{off}" if off else "")


# Timing-only builds (wrong results, never committed): python gen_lm_head_core.py now nox nobar notouch noepi leaves out the
# loop's W loads, its x loads, the barrier, the touch prefetch, the epilogue; their timings are what the design notes quote.
ABLATE = set(sys.argv[1:])
assert ABLATE <= {"now", "nox", "nobar", "notouch", "noepi"}, ABLATE


def dma_groups(stage, in_loop=False):
    """The 16 loads of one k-block into `stage` as (M0 write, load) pairs; another instruction must separate the two."""
    dst = S_DST0 if stage == 0 else S_DST1
    groups = []
    for j in range(NDMA):
        groups.append(([f"s_add_u32 m0, {dst}, {4096 * j}"], [] if (in_loop and "now" in ABLATE) else [f"global_load_lds_dwordx4 {GW[j]}, {S_WB}"]))
        groups.append(([f"s_add_u32 m0, {dst}, {TILE + 4096 * j}"], [] if (in_loop and "nox" in ABLATE) else [f"global_load_lds_dwordx4 {GX[j]}, {S_XB}"]))
    return groups


def advance_bases():
    return [f"s_add_u32 {S_WB_LO}, {S_WB_LO}, {ROW}", f"s_addc_u32 {S_WB_HI}, {S_WB_HI}, 0",
            f"s_add_u32 {S_XB_LO}, {S_XB_LO}, {ROW}", f"s_addc_u32 {S_XB_HI}, {S_XB_HI}, 0"]


def touch_ops():
    """One line of W per lane (the 256 rows of the tile over the 4 wavefronts) of a k-block that the loads will
    ask for two iterations from now, pulled into this XCD's L2 by an ordinary load whose result nobody reads: the
    loads into LDS have one iteration to land, which an L2 hit makes and a trip to HBM does not.  The touched
    k-block index saturates at the last one (touching a line twice is harmless, running off the last row is not)."""
    return ([f"v_mov_b32_e32 {DUMMY}, 0"] if "notouch" in ABLATE else [f"global_load_dword {DUMMY}, {GT}, {S_TB}"]) + [
            f"s_cmp_lt_u32 {S_TBLK}, {S_NKB1}",
            f"s_cselect_b32 {S_TMP}, {ROW}, 0",
            f"s_add_u32 {S_TB_LO}, {S_TB_LO}, {S_TMP}", f"s_addc_u32 {S_TB_HI}, {S_TB_HI}, 0",
            f"s_lshr_b32 {S_TMP}, {S_TMP}, 7", f"s_add_u32 {S_TBLK}, {S_TBLK}, {S_TMP}"]


def kstep(stage, ks, with_dma, read_next):
    """16 MFMAs of k-step ks of the k-block in `stage`.  On entry the step's 8 fragment reads are in flight (in
    READ_ORDER, nothing issued after them); on exit those of the next step are (when read_next)."""
    out = []
    half = ks & 1
    if ks == 3:
        # own reads of this k-block done, own loads of the next k-block landed; after the barrier both hold for all
        # (the newest vector-memory operation is a touch, which nobody waits for)
        out += [f"s_waitcnt vmcnt({1 if (with_dma and 'notouch' not in ABLATE) else 0}) lgkmcnt(0)"] + ([] if "nobar" in ABLATE else ["s_barrier"])
    nstage, nks = (stage, ks + 1) if ks < 3 else (1 - stage, 0)
    dma = dma_groups(stage, in_loop=True) if (ks == 3 and with_dma) else []
    issued_new = 0                                         # reads of the next step issued so far
    pos_in_order = {slot: n for n, slot in enumerate(READ_ORDER)}
    bound = 0 if ks == 3 else 8                            # upper bound of the LDS reads outstanding at this point
    for m, (vt, xt) in enumerate(MFMA_ORDER):
        if ks != 3:
            # fragments needed: W slot vt, x slot 4 + xt.  Reads complete in order, so the fragment at position
            # `need` of this step's reads has arrived once no more than (7 - need) + issued_new reads are outstanding.
            need = max(pos_in_order[vt], pos_in_order[4 + xt])
            allowed = min((7 - need) + issued_new, 15)
            if bound > allowed:
                out.append(f"s_waitcnt lgkmcnt({allowed})")
                bound = allowed
        if dma:
            out += dma[m][0]
        out.append(f"{MFMA} {acc(vt, xt)}, {frag(half, vt)}, {frag(half, 4 + xt)}, {acc(vt, xt)}")
        if read_next and m < 8:                            # early in the step: the last of them has half a step to land
            out.append(read_op(nstage, nks, 1 - half, READ_ORDER[issued_new]))
            issued_new += 1
            bound += 1
        if dma:
            out += dma[m][1]
    if dma:
        out += advance_bases() + touch_ops()
    return out


def body(stage, with_dma, last_block=False):
    out = []
    for ks in range(4):
        out += kstep(stage, ks, with_dma, read_next=not (last_block and ks == 3))
    return out


def setup():
    out = [f"v_mov_b32_e32 {NEG_INF}, 0xff800000",
           f"s_mov_b64 {S_WB}, %[wb]", f"s_mov_b64 {S_XB}, %[xb]",
           f"s_mov_b32 {S_DST0}, %[ldsw]", f"s_add_u32 {S_DST1}, %[ldsw], {STAGE}",
           f"s_mov_b32 {S_KB}, 0"]
    # load offsets: row (clamped into the tensor) * row stride + this lane's chunk
    for j in range(NDMA):
        out += [f"v_add_u32_e32 {T[0]}, {32 * j}, %[row0]",
                f"v_min_u32_e32 {T[1]}, %[wlast], {T[0]}",
                f"v_mad_u32_u24 {GW[j]}, {T[1]}, %[wsb], %[ch]",
                f"v_min_u32_e32 {T[1]}, %[xlast], {T[0]}",
                f"v_mad_u32_u24 {GX[j]}, {T[1]}, %[xsb], %[ch]"]
    # fragment addresses
    for s in range(2):
        out.append(f"v_add_u32_e32 {AW[s][0]}, {STAGE * s}, %[aw]")
        out.append(f"v_add_u32_e32 {AX[s][0]}, {STAGE * s}, %[ax]")
        for ks in range(1, 4):
            out.append(f"v_xor_b32_e32 {AW[s][ks]}, {hex(ks << 5)}, {AW[s][0]}")
            out.append(f"v_xor_b32_e32 {AX[s][ks]}, {hex(ks << 5)}, {AX[s][0]}")
    # the touch pointer starts at k-block 2 (or at the last one, if there are only two)
    out += [f"s_sub_u32 {S_NKB1}, %[nkb], 1", f"s_min_u32 {S_TBLK}, {S_NKB1}, 2", f"s_lshl_b32 {S_TMP}, {S_TBLK}, 7",
            f"s_add_u32 {S_TB_LO}, {S_WB_LO}, {S_TMP}", f"s_addc_u32 {S_TB_HI}, {S_WB_HI}, 0",
            f"v_min_u32_e32 {T[0]}, %[wlast], %[trow]",
            f"v_mul_u32_u24_e32 {GT}, %[wsb], {T[0]}"]
    # k-blocks 0 and 1 on their way
    for stage in range(2):
        for first, last in dma_groups(stage):
            out += first + ["s_nop 0"] + last
        out += advance_bases()
    # touch k-blocks 2 and 3 (saturating), leaving the touch pointer at k-block 4
    out += touch_ops() + touch_ops()
    for i in range(256):
        out.append(f"v_accvgpr_write_b32 a{i}, 0")
    out += [f"s_waitcnt vmcnt({2 * NDMA + 2})", "s_barrier"]      # k-block 0 has landed, for everybody
    for n, slot in enumerate(READ_ORDER):
        out.append(read_op(0, 0, 0, slot))
    return out


def main_loop():
    """Trips of two k-blocks (hidden % 128 == 0): all but the last trip load two k-blocks ahead."""
    out = [f"s_add_u32 {S_TMP}, {S_KB}, 2", f"s_cmp_ge_u32 {S_TMP}, %[nkb]", "s_cbranch_scc1 .Llast_%=",
           ".Ltrip_%=:"]
    out += body(0, True) + body(1, True)
    out += [f"s_add_u32 {S_KB}, {S_KB}, 2", f"s_add_u32 {S_TMP}, {S_KB}, 2", f"s_cmp_lt_u32 {S_TMP}, %[nkb]", "s_cbranch_scc1 .Ltrip_%=",
            ".Llast_%=:"]
    out += body(0, False) + body(1, False, last_block=True)
    return out


def vocab_const(e):
    i = e & 15
    return 32 * (e >> 4) + 8 * (i >> 2) + (i & 3)


def epilogue_tile(xt):
    """(max, first argmax, sum of exp) of this lane's 64 logits of x tile xt, merged over the half-wavefronts, stored."""
    C = f"%[c{xt}]"
    M, IDX, SUM, HM, MS, G = U[0], U[1], U[2], U[3], U[4], U[5]
    out = []
    for vt in range(4):
        for i in range(16):
            out.append(f"v_accvgpr_read_b32 {E[16 * vt + i]}, {acc(vt, xt, i)}")
    # the projection's output is bf16 in the reference: round to nearest even, then widen again
    for p in range(32):
        t = T[p % 4]
        out += [f"v_cvt_pk_bf16_f32 {t}, {E[2 * p]}, {E[2 * p + 1]}",
                f"v_lshlrev_b32_e32 {E[2 * p]}, 16, {t}",
                f"v_and_b32_e32 {E[2 * p + 1]}, 0xffff0000, {t}"]
    # vocabulary rows beyond the end (only the last vocab tile of the grid holds any): -inf
    out += ["s_cmp_eq_u32 %[edge], 0", f"s_cbranch_scc1 .Lnoedge{xt}_%="]
    for e in range(64):
        t = T[4 + e % 4]
        out += [f"v_add_u32_e32 {t}, {vocab_const(e)}, {VL}",
                f"v_cmp_gt_u32_e32 vcc, %[vocab], {t}",
                f"v_cndmask_b32_e32 {E[e]}, {NEG_INF}, {E[e]}, vcc"]
    out.append(f".Lnoedge{xt}_%=:")
    # maximum: two chains
    a, b = T[0], T[1]
    out += [f"v_max3_f32 {a}, {E[0]}, {E[1]}, {E[2]}", f"v_max3_f32 {b}, {E[3]}, {E[4]}, {E[5]}"]
    for e in range(6, 62, 4):
        out += [f"v_max3_f32 {a}, {a}, {E[e]}, {E[e + 1]}", f"v_max3_f32 {b}, {b}, {E[e + 2]}, {E[e + 3]}"]
    out += [f"v_max3_f32 {a}, {a}, {E[62]}, {E[63]}", f"v_max_f32_e32 {M}, {a}, {b}"]
    # first position holding it (registers ascend with the vocabulary index: descending scan, last write wins)
    out.append(f"v_mov_b32_e32 {IDX}, 0")
    for e in range(63, -1, -1):
        out += [f"v_cmp_eq_f32_e32 vcc, {E[e]}, {M}", f"v_cndmask_b32_e64 {IDX}, {IDX}, {e}, vcc"]
    # global vocabulary index of it
    out += [f"v_lshrrev_b32_e32 {T[0]}, 4, {IDX}", f"v_lshlrev_b32_e32 {T[0]}, 5, {T[0]}",            # 32 * (e >> 4)
            f"v_bfe_u32 {T[1]}, {IDX}, 2, 2", f"v_lshl_add_u32 {T[0]}, {T[1]}, 3, {T[0]}",              # + 8 * ((e >> 2) & 3)
            f"v_and_b32_e32 {T[1]}, 3, {IDX}", f"v_add3_u32 {G}, {T[0]}, {T[1]}, {VL}"]
    # sum of exp2(x c - m c): one FMA per exponent, the product m c rounded once and its error taken out afterwards
    out += [f"v_max_f32_e32 {MS}, 0xf149f2ca, {M}",                        # -1e30: keeps (-inf) - (-inf) out of the arithmetic
            f"v_mul_f32_e32 {HM}, {MS}, {C}"]
    for e0 in range(0, 64, 8):
        for e in range(e0, e0 + 8):
            out.append(f"v_fma_f32 {E[e]}, {E[e]}, {C}, -{HM}")
        for e in range(e0, e0 + 8):
            out.append(f"v_exp_f32_e32 {E[e]}, {E[e]}")
    out.append("s_nop 1")
    s4 = [U[8], U[9], U[10], U[11]]
    for k in range(4):
        out.append(f"v_add_f32_e32 {s4[k]}, {E[k]}, {E[4 + k]}")
    for e in range(8, 64, 4):
        for k in range(4):
            out.append(f"v_add_f32_e32 {s4[k]}, {s4[k]}, {E[e + k]}")
    out += [f"v_add_f32_e32 {s4[0]}, {s4[0]}, {s4[1]}", f"v_add_f32_e32 {s4[2]}, {s4[2]}, {s4[3]}",
            f"v_add_f32_e32 {SUM}, {s4[0]}, {s4[2]}",
            f"v_fma_f32 {T[0]}, {MS}, {C}, -{HM}",                          # m c - round(m c)
            f"v_exp_f32_e64 {T[0]}, -{T[0]}", "s_nop 1",
            f"v_mul_f32_e32 {SUM}, {SUM}, {T[0]}",
            # a lane all of whose logits lie beyond the vocabulary has m = -inf and a sum of 0 -- but the correction
            # factor of the stand-in maximum is 2^(+-1e22), and 0 x inf is not 0: such a lane's sum is set to 0
            f"v_cmp_lt_f32_e32 vcc, {NEG_INF}, {M}", f"v_cndmask_b32_e32 {SUM}, 0, {SUM}, vcc"]
    # merge the two half-wavefronts (lanes l and l + 32 hold the same x row): after the swaps both see both states
    M0_, M1_, S0_, S1_, G0_, G1_ = U[6], U[7], U[8], U[9], U[10], U[11]
    out += [f"v_mov_b32_e32 {M0_}, {M}", f"v_mov_b32_e32 {M1_}, {M}", f"v_mov_b32_e32 {S0_}, {SUM}", f"v_mov_b32_e32 {S1_}, {SUM}",
            f"v_mov_b32_e32 {G0_}, {G}", f"v_mov_b32_e32 {G1_}, {G}", "s_nop 1",
            f"v_permlane32_swap_b32_e32 {M0_}, {M1_}", f"v_permlane32_swap_b32_e32 {S0_}, {S1_}", f"v_permlane32_swap_b32_e32 {G0_}, {G1_}",
            "s_nop 1"]
    R_M, R_S, R_I, R_P = U[12], U[13], U[14], U[15]
    out += [f"v_max_f32_e32 {R_M}, {M0_}, {M1_}",
            f"v_max_f32_e32 {T[0]}, 0xf149f2ca, {M0_}", f"v_max_f32_e32 {T[1]}, 0xf149f2ca, {M1_}",
            f"v_max_f32_e32 {T[2]}, {T[0]}, {T[1]}",
            f"v_sub_f32_e32 {T[0]}, {T[0]}, {T[2]}", f"v_sub_f32_e32 {T[1]}, {T[1]}, {T[2]}",
            f"v_mul_f32_e32 {T[0]}, {T[0]}, {C}", f"v_mul_f32_e32 {T[1]}, {T[1]}, {C}",
            f"v_exp_f32_e32 {T[0]}, {T[0]}", f"v_exp_f32_e32 {T[1]}, {T[1]}", "s_nop 1",
            f"v_mul_f32_e32 {R_S}, {S0_}, {T[0]}", f"v_fmac_f32_e32 {R_S}, {S1_}, {T[1]}",
            f"v_min_u32_e32 {R_I}, {G0_}, {G1_}",
            f"v_cmp_gt_f32_e32 vcc, {M0_}, {M1_}", f"v_cndmask_b32_e32 {R_I}, {R_I}, {G0_}, vcc",
            f"v_cmp_gt_f32_e32 vcc, {M1_}, {M0_}", f"v_cndmask_b32_e32 {R_I}, {R_I}, {G1_}, vcc",
            f"v_mov_b32_e32 {R_P}, 0"]
    # lanes 0..31 store the record of their x row when it exists (XR is huge in lanes 32..63)
    out += [f"v_cmp_gt_u32_e32 vcc, %[rows], {XR}", "s_nop 1",
            f"s_and_saveexec_b64 {S_SAVE}, vcc",
            f"global_store_dwordx4 {PO}, v[{128 + 12}:{128 + 15}], %[pb]",
            f"s_mov_b64 exec, {S_SAVE}",
            f"v_add_u32_e32 {XR}, 32, {XR}", f"v_add_u32_e32 {PO}, %[postep], {PO}"]
    return out


def epilogue():
    if "noepi" in ABLATE:
        return ["s_nop 15", "s_waitcnt vmcnt(0)"]
    out = ["s_nop 15", "s_nop 15", "s_nop 15", "s_nop 15", "s_nop 15",
           f"v_mov_b32_e32 {PO}, %[po]", f"v_mov_b32_e32 {XR}, %[xrow]", f"v_mov_b32_e32 {VL}, %[vlane]"]
    for xt in range(4):
        out += epilogue_tile(xt)
    out.append("s_waitcnt vmcnt(0)")
    return out


def program():
    return setup() + main_loop() + epilogue()


HEADER = '''// GENERATED by gen_lm_head_core.py -- do not edit; change the generator and regenerate.
//
// Core of the fused vocabulary projection + confidence reduction (see the generator's docstring for the
// schedule, the LDS layout and the register map).  Everything between the first load of W / x and the stores
// of the per-slice records happens inside this one asm statement; the physical registers it uses are
// declared as clobbers, the operands are read-only.
struct LmHeadCoreArgs {
    unsigned aw, ax;                 // per-lane LDS byte address of this lane's W / x fragment of k-step 0, tile 0, stage 0
    unsigned row0;                   // row of the 256-row tile that this lane loads first (then 32 further down, 8 times)
    unsigned trow;                   // row of the W tile whose lines this lane touches ahead of the loads (thread index)
    unsigned ch;                     // byte offset inside a 128-byte k-block row of the 16-byte chunk this lane loads
    unsigned wlast, xlast;           // last valid row of the W / x tile (rows beyond are clamped onto it)
    unsigned wsb, xsb;               // bytes between consecutive rows of W / x
    const void* wb; const void* xb;  // first row of this workgroup's W / x tile
    unsigned ldsw;                   // LDS byte address of the first row this wavefront loads in stage 0's W tile
    unsigned nkb;                    // k-blocks of 64 (even)
    float c0, c1, c2, c3;            // log2(e) / temperature of this lane's x row in x tiles 0..3
    unsigned vlane;                  // vocabulary index of this lane's first accumulator register
    unsigned vocab, edge;            // vocabulary size; non-zero when this tile reaches beyond it
    unsigned xrow;                   // this lane's x row in x tile 0 (lanes 32..63: 0x7fffffff, they store nothing)
    unsigned rows;                   // x rows in all
    const void* pb;                  // records: 16 bytes (max, sum, argmax, 0) each
    unsigned po, postep;             // byte offset of this lane's record of x tile 0; step per x tile
};

__device__ __forceinline__ void lm_head_core(const LmHeadCoreArgs& A)
{
    asm volatile(
'''


def main():
    prog = program()
    text = "\n".join(f'        "{line}\\n"' for line in prog)
    vclob = ", ".join(f'"v{r}"' for r in range(16, 256))
    aclob = ", ".join(f'"a{r}"' for r in range(256))
    sclob = ", ".join(f'"s{r}"' for r in range(40, 60))
    tail = f'''
        :
        : [aw] "v"(A.aw), [ax] "v"(A.ax), [row0] "v"(A.row0), [trow] "v"(A.trow), [ch] "v"(A.ch),
          [c0] "v"(A.c0), [c1] "v"(A.c1), [c2] "v"(A.c2), [c3] "v"(A.c3),
          [vlane] "v"(A.vlane), [xrow] "v"(A.xrow), [po] "v"(A.po),
          [wlast] "s"(A.wlast), [xlast] "s"(A.xlast), [wsb] "s"(A.wsb), [xsb] "s"(A.xsb),
          [wb] "s"(A.wb), [xb] "s"(A.xb), [ldsw] "s"(A.ldsw), [nkb] "s"(A.nkb),
          [vocab] "s"(A.vocab), [edge] "s"(A.edge), [rows] "s"(A.rows), [pb] "s"(A.pb), [postep] "s"(A.postep)
        : "memory", "vcc", "scc", "m0", {sclob},
          {vclob},
          {aclob});
}}
'''
    sys.stdout.write(HEADER + text + tail)
    sys.stderr.write(f"{len(prog)} instructions\n")


if __name__ == "__main__":
    main()
