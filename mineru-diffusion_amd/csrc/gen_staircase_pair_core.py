#!/usr/bin/env python3
"""Generator of staircase_pair_core.inc: the hand-scheduled gfx950 key loop of the staircase
block-prefill attention kernel for a PAIR of query heads that share a KV head.

Run  python gen_staircase_pair_core.py > staircase_pair_core.inc  after changing the schedule; the
.inc file is what the build compiles.

Why assembly: one wavefront per SIMD has to keep the MFMA pipe busy by itself.  Instructions of one
wavefront issue in order, so LDS fragment reads must run several fragments ahead of the MFMA that
consumes them and the softmax arithmetic of tile t has to be issued in the shadow of the MFMAs of
tile t+1.  Both need exact control of instruction order and of physical registers that persist
across loop iterations, which neither the compiler's scheduler nor inline-asm operands (no
sub-register access to a 16-register tuple) offer.

Work of one wavefront: 32 query rows x 2 heads, keys in tiles of 64.
  S'^T[key, q] = K . (c Q)^T - m    A = K fragment (LDS, ds_read_b128), B = scaled Q^T (accumulation
                                    registers), C = a tuple holding -m (the stale running max)
  P = exp2(S'), bf16, in place
  O^T[d, q]  += V^T . P^T           A = V^T fragment (LDS, two ds_read_b64_tr_b16), B = P^T
Every K / V^T fragment feeds the MFMAs of both heads.  Register and key maps are those of
attn_tile.h (key_of_reg, key_of_mfma_row).

LDS: five slots of 32 KB (tile % 5), K rows then V rows, 256 bytes per row, filled by
global_load_lds_dwordx4 (1 KB = 4 rows per instruction, 8 instructions per wavefront and tile).  The
16-byte chunk c of row r sits at position c ^ (r % 16), which makes both fragment read patterns
bank-conflict free without padding; the XOR shows up as one address register per k-step.

Loop iteration t (S is double-buffered, cb = t & 1).  The MFMA / fragment stream never drains: the
reads of the first fragments of iteration t+1 are issued during the last items of iteration t.
  items 0..15:  32 MFMAs of QK(t+1) -> S[1-cb]   ||  rescale check(t), P(t) = exp2(S[cb]) in place
  wait until tile t+2 (loaded two iterations ago) has landed, barrier (publishes it; everyone has left tile t-1)
  items 16..31: 32 MFMAs of PV(t) + 16 small ones (row sums)    ||  loads of tile t+4 -> slot of
                tile t-1, row max of S[1-cb], fragment addresses of iteration t+1, addresses of tile t+5

Physical registers (all clobbered; the compiler keeps v0..v15 and a128..a191, a224..a255 for operands):
  v16..v23  temporaries                  v24..v39  K / V^T fragment addresses
  v40..v63  state, ones, load addresses  v64..v191 S[2][head][sub-tile][16]
  v192..v223 -m tuples                   v224..v255 fragment ring (8 x 4)
  a0..a127  O^T[head][d tile][16]        a192..a223 row sums            s40..s55 loop state
"""
import sys

# Element type of q / k / v / o: "bf16" (default) or "f16" (python gen_staircase_pair_core.py f16).  The two cores differ
# in the MFMA mnemonics, the bit pattern of 1.0 and the float -> element conversions: probabilities are packed by one
# instruction either way (round to nearest even for bf16; fp16 has only the round-toward-zero pack, whose bias the
# row sums share, since they are taken from the packed values), the output is rounded to nearest even in both.
DT = sys.argv[1] if len(sys.argv) > 1 else "bf16"
assert DT in ("bf16", "f16")
MFMA = f"v_mfma_f32_32x32x16_{DT}"
MFMA_SUM = f"v_mfma_f32_4x4x4_16b_{DT}"
ONE_PAIR = "0x3f803f80" if DT == "bf16" else "0x3c003c00"
CVT_P = "v_cvt_pk_bf16_f32" if DT == "bf16" else "v_cvt_pkrtz_f16_f32"

ROW = 256
K_BYTES = 64 * ROW                 # 16384: K part of a slot; V part follows
SLOT = 2 * K_BYTES
RING_SLOTS = 8
RING_DEPTH = 6                     # fragments in flight
DMA_PER_TILE = 8                   # global_load_lds instructions per wavefront and tile

# ---- register names ---------------------------------------------------------------------------
KA = [f"v{24 + i}" for i in range(8)]            # K fragment address of k-step ks (current slot)
VA = [[f"v{32 + 4 * q + dt}" for dt in range(4)] for q in range(2)]   # V^T address [lo / hi][d tile]
VPAD, VLPM1, JPL, NEG_INF = "v40", "v41", "v42", "v43"
ONES = "v[52:53]"                                # four bf16 ones: A operand of the row-sum MFMA (see lacc)
MX = ["v48", "v49"]
MREL = "v50"
GK = [f"v{56 + i}" for i in range(4)]            # global byte offsets of the rows the next loads fetch
GV = [f"v{60 + i}" for i in range(4)]
T = [f"v{16 + i}" for i in range(8)]
S_T, S_KEY0, S_R0, S_R1, S_R2, S_R3, S_TMP = "s40", "s41", "s42", "s43", "s44", "s45", "s46"
S_R4 = "s51"
S_SAVE = "s[48:49]"
S_DST = "s50"


def sreg(b, h, u, i):
    return 64 + 64 * b + 32 * h + 16 * u + i


def stup(b, h, u):
    r = sreg(b, h, u, 0)
    return f"v[{r}:{r + 15}]"


def ptup(b, h, u, t):
    r = sreg(b, h, u, 8 * t)
    return f"v[{r}:{r + 3}]"


def phalf(b, h, u, t, half):
    r = sreg(b, h, u, 8 * t) + 2 * half
    return f"v[{r}:{r + 1}]"


def negm(h, i=None):
    r = 192 + 16 * h
    return f"v[{r}:{r + 15}]" if i is None else f"v{r + i}"


def otup(h, dt):
    r = 64 * h + 16 * dt
    return f"a[{r}:{r + 15}]"


L_REGS = 4


def lacc(h, i=None):
    """Row sums l of head h.  v_mfma_f32_4x4x4_16b_bf16 with A = ones adds, in every lane, the lane's own
    four B values to each of its four accumulator registers (16 independent 4x4 blocks of four lanes:
    D[i][j] = sum_k B[k][j], and lane 4 b + j holds column j of block b in A, B and D alike).  A lane's P^T
    operands all belong to its one query, so this is the horizontal add that the row sum needs, on the
    matrix pipe, at 8 cycles per four values: 16 of them per 64-key tile (128 cycles) where multiplying
    the 32x32x16 operands by a block of ones took 8 x 32 cycles.  Each lane sums the keys of its own half
    of every k-step; the two halves of a query (lanes l and l + 32) are added in the epilogue."""
    r = 192 + 16 * h
    return f"a[{r}:{r + L_REGS - 1}]" if i is None else f"a{r + i}"


def ring(i):
    r = 224 + 4 * (i % RING_SLOTS)
    return f"v[{r}:{r + 3}]", f"v[{r}:{r + 1}]", f"v[{r + 2}:{r + 3}]"


# ---- VALU fragments -----------------------------------------------------------------------------
def key_const(u, i):
    return 32 * u + 16 * (i >> 3) + 4 * (i & 3) + ((i >> 2) & 1)


def softmax_plan(cb, masked):
    """S[cb] -> P in place, both heads, in the order PV consumes it, as {item: [ops]}.
    P(h, u, t) = chunk c = 2(2u + t) + h (8 values) is first read by PV item 16 + 4(2u + t).  The QK
    items are the busy ones (two MFMAs, a fragment read and their share of these instructions have
    to issue within the 65 cycles the two MFMAs execute), the PV items have room: chunks 0..5 are
    exponentiated three values per QK item, chunks 6, 7 (read from item 28 on) during PV items
    16..19; a chunk is converted at least one item after its last exponential (a v_exp result needs
    a gap before another kind of instruction reads it), chunks 4..7 during PV items.  The row sums
    are not computed here: the PV part multiplies P^T by a fragment of ones (8 MFMAs per tile
    instead of 64 adds, or 32 v_dot2, which execute on the matrix pipe and stall the MFMAs they
    are meant to hide behind)."""
    plan = {n: [] for n in range(32)}
    chunks = [(h, u, t) for u in range(2) for t in range(2) for h in range(2)]

    def exp_ops(c, j):
        h, u, t = chunks[c]
        r = sreg(cb, h, u, 8 * t + j)
        ops = []
        if masked:
            # temporaries T[4..7]: the row maximum of the other tile accumulates in T[0..3] during items 18..25,
            # which overlap the last of these (items 16..19)
            ops += [f"v_add_u32_e32 {T[4 + j % 4]}, {key_const(u, 8 * t + j)}, {MREL}",
                    f"v_cmp_lt_u32_e32 vcc, {T[4 + j % 4]}, %[mlim]",
                    f"v_cndmask_b32_e32 v{r}, {NEG_INF}, v{r}, vcc"]
        return ops + [f"v_exp_f32_e32 v{r}, v{r}"]

    def cvt_op(c, j):
        h, u, t = chunks[c]
        base = sreg(cb, h, u, 8 * t)
        return f"{CVT_P} v{base + j}, v{base + 2 * j}, v{base + 2 * j + 1}"

    last_exp_item = {}
    for e in range(48):                               # chunks 0..5: three values per QK item
        c, j = e >> 3, e & 7
        plan[e // 3] += exp_ops(c, j)
        last_exp_item[c] = e // 3
    for e in range(16):                               # chunks 6, 7: four values per item 16..19
        c, j = 6 + (e >> 3), e & 7
        plan[16 + e // 4] += exp_ops(c, j)
        last_exp_item[c] = 16 + e // 4
    for c in range(8):
        first = {4: 16, 5: 17, 6: 20, 7: 21}.get(c, last_exp_item[c] + 1)
        assert first > last_exp_item[c] and first + 1 < 16 + 4 * (c >> 1)
        for j in range(4):
            plan[first + (j >> 1)].append(cvt_op(c, j))
    return plan


def rowmax_ops(b):
    """MX[h] = max over this query's 64 keys of S[b][h] (both half-waves); the two heads' chains
    alternate so that no instruction depends on its predecessor."""
    ops = []
    regs = {h: [sreg(b, h, u, i) for u in range(2) for i in range(16)] for h in range(2)}
    acc = {h: (T[2 * h], T[2 * h + 1]) for h in range(2)}
    for h in range(2):
        ops.append(f"v_max3_f32 {acc[h][0]}, v{regs[h][0]}, v{regs[h][1]}, v{regs[h][2]}")
    for h in range(2):
        ops.append(f"v_max3_f32 {acc[h][1]}, v{regs[h][3]}, v{regs[h][4]}, v{regs[h][5]}")
    for i in range(6, 32, 2):
        for h in range(2):
            d = acc[h][(i >> 1) & 1]
            ops.append(f"v_max3_f32 {d}, {d}, v{regs[h][i]}, v{regs[h][i + 1]}")
    for h in range(2):
        ops.append(f"v_max_f32_e32 {acc[h][0]}, {acc[h][0]}, {acc[h][1]}")
    for h in range(2):
        ops.append(f"v_mov_b32_e32 {acc[h][1]}, {acc[h][0]}")
    ops.append("s_nop 1")
    for h in range(2):
        ops.append(f"v_permlane32_swap_b32_e32 {acc[h][0]}, {acc[h][1]}")
    ops.append("s_nop 1")
    for h in range(2):
        ops.append(f"v_max_f32_e32 {MX[h]}, {acc[h][0]}, {acc[h][1]}")
    return ops


def load_offset_ops():
    """Byte offsets of the rows the next global loads fetch (rows clamped into the sequence), then JPL += 64."""
    ops = []
    for i in range(4):
        ops.append(f"v_add_u32_e32 {T[6]}, {16 * i}, {JPL}")
        ops.append(f"v_med3_i32 {T[6]}, {T[6]}, {VPAD}, {VLPM1}")
        ops.append(f"v_mad_u32_u24 {GK[i]}, {T[6]}, %[krb], %[ch]")
        ops.append(f"v_mad_u32_u24 {GV[i]}, {T[6]}, %[vrb], %[ch]")
    ops.append(f"v_add_u32_e32 {JPL}, 64, {JPL}")
    return ops


def dma_ops(slot_sreg):
    """The 8 global -> LDS loads of one tile into the slot whose byte offset is in slot_sreg, as
    (M0 write, load) pairs: M0 = LDS destination of lane 0; other instructions must separate the two."""
    groups = []
    for i in range(4):
        for kv, (off, base) in enumerate(((GK, "%[kb]"), (GV, "%[vb]"))):
            first = [f"s_add_u32 m0, {S_DST}, {4096 * i + K_BYTES * kv}"]
            if i == 0 and kv == 0:
                first = [f"s_add_u32 {S_DST}, {slot_sreg}, %[wrow]"] + first
            groups.append((first, [f"global_load_lds_dwordx4 {off[i]}, {base}"]))
    return groups


def k_address_ops(slot_sreg):
    """K fragment addresses (one per k-step: the swizzle is an XOR) for the slot in slot_sreg."""
    ops = [f"v_add_u32_e32 {KA[0]}, {slot_sreg}, %[ka]"]
    for ks in range(1, 8):
        ops.append(f"v_xor_b32_e32 {KA[ks]}, {hex(ks << 5)}, {KA[0]}")
    return ops


def v_address_ops(slot_sreg):
    """V^T fragment addresses (two rows x four d tiles) for the slot in slot_sreg."""
    ops = []
    for q, name in enumerate(("%[val]", "%[vah]")):
        ops.append(f"v_add_u32_e32 {VA[q][0]}, {slot_sreg}, {name}")
        for dt in range(1, 4):
            ops.append(f"v_xor_b32_e32 {VA[q][dt]}, {hex(dt << 6)}, {VA[q][0]}")
    return ops


def mask_ops(b):
    """S[b] value -> -inf wherever its key is not visible to this lane's query (the test of the
    exponential's mask; applying it twice is harmless)."""
    ops = []
    for h in range(2):
        for u in range(2):
            for i in range(16):
                r = sreg(b, h, u, i)
                ops += [f"v_add_u32_e32 {T[i % 4]}, {key_const(u, i)}, {MREL}",
                        f"v_cmp_lt_u32_e32 vcc, {T[i % 4]}, %[mlim]",
                        f"v_cndmask_b32_e32 v{r}, {NEG_INF}, v{r}, vcc"]
    return ops


def check_rescale(uid, cb, masked):
    """Lazy running-max update from MX = row max of S' = c s - m: only when some query of either
    head exceeds the stale max by more than 2^8.  The rare path moves m up by delta = max(MX, 0):
    the -m tuple and the scores of tile t (computed with the old m) go down by delta, the row sums
    and O^T (accumulation registers) are scaled by 2^-delta.
    MX was taken over all 64 keys of the tile, visible or not: an upper bound of the visible maximum,
    good enough to decide that nothing has to move.  When something may have to move and the tile
    holds keys that some query must not see, the maximum is taken again over the visible keys only:
    a hidden key with a score far above every visible one must not raise m (the visible terms, and
    everything accumulated so far, would be scaled to zero)."""
    lab = f".Lskip_{uid}_%="
    out = [f"v_max_f32_e32 {T[0]}, {MX[0]}, {MX[1]}",
           f"v_cmp_lt_f32_e32 vcc, 0x41000000, {T[0]}",
           f"s_cbranch_vccz {lab}"]
    if masked:
        out += mask_ops(cb) + rowmax_ops(cb)
    for h in range(2):
        out.append(f"v_max_f32_e32 {T[0]}, 0, {MX[h]}")
        out.append(f"v_exp_f32_e64 {T[1]}, -{T[0]}")
        for i in range(16):
            out.append(f"v_sub_f32_e32 {negm(h, i)}, {negm(h, i)}, {T[0]}")
        for u in range(2):
            for i in range(16):
                r = sreg(cb, h, u, i)
                out.append(f"v_sub_f32_e32 v{r}, v{r}, {T[0]}")
        out.append("s_nop 15")                      # the MFMAs of the previous tile's PV have long finished; margin only
        for i in range(64 + L_REGS):
            a = f"a{64 * h + i}" if i < 64 else lacc(h, i - 64)
            t = T[2 + (i & 3)]
            out.append(f"v_accvgpr_read_b32 {t}, {a}")
            out.append(f"v_mul_f32_e32 {t}, {t}, {T[1]}")
            out.append(f"v_accvgpr_write_b32 {a}, {t}")
    out.append("s_nop 7")
    out.append(f"{lab}:")
    return out


# ---- MFMA / fragment stream ----------------------------------------------------------------------
def qk_items(nb):
    """K fragment n = (u = n & 1, ks = n >> 1) -> S[nb][h][u] for h = 0, 1."""
    items = []
    for n in range(16):
        u, ks = n & 1, n >> 1
        rd = lambda frag, u=u, ks=ks: [f"ds_read_b128 {frag[0]}, {KA[ks]}" + (f" offset:{u * 32 * ROW}" if u else "")]
        mf = lambda frag, u=u, ks=ks: [
            f"{MFMA} {stup(nb, h, u)}, {frag[0]}, %[q{h}{ks}], {negm(h) if ks == 0 else stup(nb, h, u)}"
            for h in range(2)]
        items.append((rd, mf))
    return items


def pv_items(cb):
    """V^T fragment m = (u, t, dt) = (m >> 3, (m >> 2) & 1, m & 3); O^T[h][dt] += fragment . P[h][u][t]."""
    items = []
    for m in range(16):
        u, t, dt = m >> 3, (m >> 2) & 1, m & 3
        o = (u * 32 + t * 16) * ROW
        sfx = f" offset:{o}" if o else ""
        rd = lambda frag, dt=dt, sfx=sfx: [f"ds_read_b64_tr_b16 {frag[1]}, {VA[0][dt]}{sfx}",
                                           f"ds_read_b64_tr_b16 {frag[2]}, {VA[1][dt]}{sfx}"]
        mf = lambda frag, u=u, t=t, dt=dt: [
            f"{MFMA} {otup(h, dt)}, {frag[0]}, {ptup(cb, h, u, t)}, {otup(h, dt)}" for h in range(2)] + (
            [f"{MFMA_SUM} {lacc(h)}, {ONES}, {phalf(cb, h, u, t, half)}, {lacc(h)}"
             for half in range(2) for h in range(2)] if dt == 1 else [])
        items.append((rd, mf))
    return items


class Ring:
    """Issue order of the fragment reads and the exact lgkmcnt value that waits for one of them
    (LDS operations of a wavefront complete in order; nothing else uses that counter here)."""

    def __init__(self):
        self.issued = 0
        self.last = {}

    def read(self, out, key, item, slot_index):
        for r in item[0](ring(slot_index)):
            out.append(r)
            self.issued += 1
        self.last[key] = self.issued - 1

    def wait(self, out, key):
        w = self.issued - 1 - self.last[key]
        assert 0 <= w <= 15, w
        out.append(f"s_waitcnt lgkmcnt({w})")


def spread(out, mfmas, valu):
    """MFMAs of one item with its other instructions dealt evenly behind them."""
    base, rem = divmod(len(valu), len(mfmas))
    k = 0
    for i, m in enumerate(mfmas):
        out.append(m)
        c = base + (1 if i < rem else 0)
        out.extend(valu[k:k + c])
        k += c


def qk0_block(out):
    """Prologue: QK(0) with C = 0 -> S[0]; drains its reads."""
    items = qk_items(0)
    rg = Ring()
    for n in range(RING_DEPTH):
        rg.read(out, n, items[n], n)
    for n in range(16):
        rg.wait(out, n)
        for m in items[n][1](ring(n)):
            out.append(m.replace(f", {negm(0)}", ", 0").replace(f", {negm(1)}", ", 0"))
        if n + RING_DEPTH < 16:
            rg.read(out, n + RING_DEPTH, items[n + RING_DEPTH], n + RING_DEPTH)


def prologue():
    out = []
    out += [f"v_mov_b32_e32 {NEG_INF}, 0xff800000", f"v_mov_b32_e32 {VPAD}, %[pad]", f"v_mov_b32_e32 {VLPM1}, %[lpm1]",
            f"v_mov_b32_e32 {MREL}, %[mrel]", f"v_mov_b32_e32 {JPL}, %[jpl]"]
    out += [f"s_mov_b32 {S_T}, 0", f"s_mov_b32 {S_KEY0}, 0", f"s_mov_b32 {S_R0}, 0", f"s_mov_b32 {S_R1}, {SLOT}",
            f"s_mov_b32 {S_R2}, {2 * SLOT}", f"s_mov_b32 {S_R3}, {3 * SLOT}", f"s_mov_b32 {S_R4}, {4 * SLOT}"]
    # tiles 0..3 -> slots 0..3; addresses of tile 4 prepared
    for slot in (S_R0, S_R1, S_R2, S_R3):
        out += load_offset_ops()
        for first, last in dma_ops(slot):
            out += first + ["s_nop 0"] + last
    out += load_offset_ops()
    for i in range(2):
        out.append(f"v_mov_b32_e32 v{52 + i}, {ONE_PAIR}")
    for i in list(range(128)) + [192 + 16 * h + j for h in range(2) for j in range(L_REGS)]:
        out.append(f"v_accvgpr_write_b32 a{i}, 0")
    out += [f"s_waitcnt vmcnt({2 * DMA_PER_TILE})", "s_barrier"]      # tiles 0 and 1 have landed
    # QK(0) with C = 0, then m = row max of tile 0: -m tuples and S[0] -= m
    out += k_address_ops(S_R0)
    qk0_block(out)
    out.append("s_nop 15")
    # m starts as the maximum over the keys each query may see: when the wavefront's first limit lies
    # inside tile 0 the hidden keys are taken out first (keys before the sequence are copies of its
    # first key, which every query sees: they cannot raise the maximum)
    out += [f"s_movk_i32 {S_TMP}, 64", f"s_cmp_gt_i32 {S_TMP}, %[whm]", "s_cbranch_scc0 .Lplain0_%="]
    out += mask_ops(0)
    out.append(".Lplain0_%=:")
    out += rowmax_ops(0)
    for h in range(2):
        for i in range(16):
            out.append(f"v_sub_f32_e32 {negm(h, i)}, 0, {MX[h]}")
        for u in range(2):
            for i in range(16):
                r = sreg(0, h, u, i)
                out.append(f"v_sub_f32_e32 v{r}, v{r}, {MX[h]}")
        out.append(f"v_mov_b32_e32 {MX[h]}, 0")
    # iteration 0 starts with its first K fragments (tile 1) in flight
    out += k_address_ops(S_R1) + v_address_ops(S_R0)
    items = qk_items(1)
    for n in range(RING_DEPTH):
        out += items[n][0](ring(n))
    return out


def body(cb, masked):
    """One iteration.  On entry the reads of items 0..RING_DEPTH-1 are in flight; on exit those of
    the next iteration are."""
    uid = f"{cb}{int(masked)}"
    out = []
    nb = 1 - cb
    items = qk_items(nb) + pv_items(cb)
    nxt = qk_items(cb)                                  # only their reads are used: first fragments of iteration t+1
    plan = softmax_plan(cb, masked)
    # second half: K addresses of tile t+2 (the K reads of this iteration were all issued by item 9),
    # row max of S[nb] (complete after item 15), V^T addresses of tile t+1 (after the last V^T read
    # of this iteration has been issued, item 25), addresses of the loads of tile t+4 (after the
    # loads of tile t+3, items 17..24)
    ka2 = k_address_ops(S_R2)
    for i, op in enumerate(ka2):
        plan[16 + i].append(op)
    rm = rowmax_ops(nb)
    per = -(-len(rm) // 8)
    for i in range(8):
        plan[18 + i] += rm[per * i:per * (i + 1)]
    tail = v_address_ops(S_R1) + load_offset_ops()
    per = -(-len(tail) // 6)
    for i in range(6):
        plan[26 + i] += tail[per * i:per * (i + 1)]
    dma = dma_ops(S_R4)
    rg = Ring()
    for n in range(RING_DEPTH):
        rg.last[n] = n
    rg.issued = RING_DEPTH
    out += check_rescale(uid, cb, masked)
    for n in range(32):
        if n == 16:
            # tile t+2 (loaded two iterations ago; tile t+3 may still be in flight) has landed; after
            # the barrier every wavefront sees it and has left tile t-1, whose slot the loads below
            # (tile t+4) overwrite
            out += [f"s_waitcnt vmcnt({DMA_PER_TILE})", "s_barrier"]
        if n % 2 == 0:
            rg.wait(out, n + 1)
        first, last = dma[n - 17] if 17 <= n < 17 + DMA_PER_TILE else ([], [])
        out.extend(first)
        spread(out, items[n][1](ring(n)), plan[n])
        k = n + RING_DEPTH
        rg.read(out, k, items[k] if k < 32 else nxt[k - 32], k)
        out.extend(last)
    out += [f"s_mov_b32 {S_TMP}, {S_R0}", f"s_mov_b32 {S_R0}, {S_R1}", f"s_mov_b32 {S_R1}, {S_R2}", f"s_mov_b32 {S_R2}, {S_R3}",
            f"s_mov_b32 {S_R3}, {S_R4}", f"s_mov_b32 {S_R4}, {S_TMP}",
            f"s_add_i32 {S_T}, {S_T}, 1", f"s_add_i32 {S_KEY0}, {S_KEY0}, 64", f"v_add_u32_e32 {MREL}, 64, {MREL}"]
    return out


def body_last(cb):
    """The iteration of the last tile that holds keys this wavefront may see: softmax and PV of tile t as in the
    masked body, but no QK of tile t+1 (every one of its probabilities would be zero: the half of an ordinary
    iteration's matrix work that the wavefront's first hidden tile used to cost).  The K fragment reads that the
    previous iteration issued ahead are left to land unused.  Leaves into the idle loop."""
    uid = f"{cb}L"
    out = []
    items = [None] * 16 + pv_items(cb)
    plan = softmax_plan(cb, True)
    tail = load_offset_ops()
    per = -(-len(tail) // 6)
    for i in range(6):
        plan[26 + i] += tail[per * i:per * (i + 1)]
    dma = dma_ops(S_R4)
    rg = Ring()
    rg.issued = RING_DEPTH                              # the K reads in flight on entry: they complete first, in order
    out += check_rescale(uid, cb, True)
    out += v_address_ops(S_R0)                          # V^T addresses of tile t (the previous iteration set them too; kept explicit)
    for n in range(32):
        if n == 16:
            out += [f"s_waitcnt vmcnt({DMA_PER_TILE})", "s_barrier"]
        if n < 16:
            out.extend(plan[n])
            out.append("s_nop 1")                       # no MFMAs here to space a v_exp from the conversion that reads it
            k = n + RING_DEPTH
            if k >= 16:
                rg.read(out, k, items[k], k)
            continue
        if n % 2 == 0:
            rg.wait(out, n + 1)
        first, last = dma[n - 17] if 17 <= n < 17 + DMA_PER_TILE else ([], [])
        out.extend(first)
        spread(out, items[n][1](ring(n)), plan[n])
        k = n + RING_DEPTH
        if k < 32:
            rg.read(out, k, items[k], k)
        out.extend(last)
    out += [f"s_mov_b32 {S_TMP}, {S_R0}", f"s_mov_b32 {S_R0}, {S_R1}", f"s_mov_b32 {S_R1}, {S_R2}", f"s_mov_b32 {S_R2}, {S_R3}",
            f"s_mov_b32 {S_R3}, {S_R4}", f"s_mov_b32 {S_R4}, {S_TMP}",
            f"s_add_i32 {S_T}, {S_T}, 1",
            f"s_cmp_ge_i32 {S_T}, %[nt]",
            "s_cbranch_scc1 .Lend_%=",
            "s_branch .Lidle_%="]
    return out


def select(cb):
    """Top of iteration t: leave after the last tile; tiles that need the key mask go out of line."""
    return [f".Ltop_{cb}_%=:",
            f"s_cmp_ge_i32 {S_T}, %[nt]",
            "s_cbranch_scc1 .Lend_%=",
            f"s_cmp_ge_i32 {S_KEY0}, %[whx]",
            "s_cbranch_scc1 .Lidle_%=",
            f"s_add_i32 {S_TMP}, {S_KEY0}, 64",
            f"s_cmp_ge_i32 {S_TMP}, %[whx]",
            f"s_cbranch_scc1 .Llast_{cb}_%=",
            f"s_cmp_lt_i32 {S_KEY0}, %[pad]",
            f"s_cbranch_scc1 .Lmasked_{cb}_%=",
            f"s_cmp_gt_i32 {S_TMP}, %[whm]",
            f"s_cbranch_scc1 .Lmasked_{cb}_%="]


def idle_loop():
    """Iterations whose tile lies wholly beyond the last key that any query of this wavefront may see (the other
    wavefronts of the workgroup own later rows and still need the tile): nothing to compute -- every probability
    would be zero -- but the wavefront keeps loading its quarter of every tile and meets the others at the barrier.
    Entered from the top of an iteration, left only through the end of the loop."""
    out = [".Lidle_%=:",
           f"s_waitcnt vmcnt({DMA_PER_TILE})", "s_barrier"]
    for first, last in dma_ops(S_R4):
        out += first + ["s_nop 0"] + last
    out += load_offset_ops()
    out += [f"s_mov_b32 {S_TMP}, {S_R0}", f"s_mov_b32 {S_R0}, {S_R1}", f"s_mov_b32 {S_R1}, {S_R2}", f"s_mov_b32 {S_R2}, {S_R3}",
            f"s_mov_b32 {S_R3}, {S_R4}", f"s_mov_b32 {S_R4}, {S_TMP}",
            f"s_add_i32 {S_T}, {S_T}, 1",
            f"s_cmp_ge_i32 {S_T}, %[nt]",
            "s_cbranch_scc0 .Lidle_%="]
    return out


def epilogue():
    """O = O^T / l as bf16 rows.  The accumulators hold O transposed (a lane has 4 consecutive d of its query per
    d group): stored from there, a store instruction touches 32 rows with 16 bytes each.  Instead every wavefront
    turns its 32 x 128 tile of one head around through 8 KB of LDS and writes whole rows: 16 lanes x 16 bytes per
    row, four rows per instruction, 8 instructions per head (before: 16 of half the width, and they cost a tenth
    of a launch of 1000-token sequences).  The LDS comes from the slot of tile nt + 1: that tile was loaded ahead
    of need and landed, for every wavefront, before the barrier of the last iteration; nobody reads it and no
    load still in flight targets it (those are tiles nt + 2 and nt + 3).  Rows use the K / V swizzle (16-byte
    chunk c of row r at position c ^ (r % 16)), which keeps the 8-byte writes of a (d tile, group) off each
    other's banks; the reads are linear."""
    LN, X, WB, RB, L4, OFFL, C0, RV = (f"v{80 + i}" for i in range(8))
    WA = [f"v{64 + c}" for c in range(16)]
    SO = [f"v{88 + m}" for m in range(4)]
    TMP = [f"v{92 + i}" for i in range(2)]
    OFFJ = [f"v{94 + i}" for i in range(2)]
    S_STEP = "s47"
    out = [".Lend_%=:", "s_waitcnt lgkmcnt(0)", "s_nop 15", "s_nop 15"]
    out += [f"v_mbcnt_lo_u32_b32 {LN}, -1, 0", f"v_mbcnt_hi_u32_b32 {LN}, -1, {LN}",
            f"v_and_b32_e32 {X}, 15, {LN}", f"v_lshlrev_b32_e32 {X}, 4, {X}",
            f"v_and_b32_e32 {TMP[0]}, 31, {LN}", f"v_lshlrev_b32_e32 {TMP[0]}, 8, {TMP[0]}",
            f"v_lshrrev_b32_e32 {TMP[1]}, 5, {LN}", f"v_lshl_add_u32 {TMP[0]}, {TMP[1]}, 3, {TMP[0]}",
            f"s_add_u32 {S_TMP}, {S_R1}, %[owave]",
            f"v_add_u32_e32 {WB}, {S_TMP}, {TMP[0]}",
            f"v_lshl_add_u32 {RB}, {LN}, 4, {S_TMP}",
            f"v_lshrrev_b32_e32 {L4}, 4, {LN}",
            f"v_mul_lo_u32 {OFFL}, {L4}, %[ostb]",
            f"v_lshlrev_b32_e32 {TMP[0]}, 4, {L4}", f"v_xor_b32_e32 {C0}, {TMP[0]}, {X}",
            f"v_add_u32_e32 {RV}, %[orow0], {L4}"]
    for c in range(16):
        out += [f"v_xor_b32_e32 {WA[c]}, {16 * c}, {X}", f"v_add_u32_e32 {WA[c]}, {WA[c]}, {WB}"]
    for m in range(4):
        out += [f"v_xor_b32_e32 {SO[m]}, {64 * m}, {C0}", f"v_add_u32_e32 {SO[m]}, {SO[m]}, {OFFL}"]
    for h in range(2):
        data = [f"v[{96 + 32 * h + 4 * j}:{96 + 32 * h + 4 * j + 3}]" for j in range(8)]
        # l = this lane's partial sum + that of the lane holding the other keys of the same query
        out += [f"v_accvgpr_read_b32 {T[7]}, {lacc(h, 0)}", "s_nop 1", f"v_mov_b32_e32 {T[6]}, {T[7]}", "s_nop 1",
                f"v_permlane32_swap_b32_e32 {T[7]}, {T[6]}", "s_nop 1",
                f"v_add_f32_e32 {T[7]}, {T[7]}, {T[6]}", f"v_rcp_f32_e32 {T[7]}, {T[7]}", "s_nop 0"]
        for dt in range(4):
            for g in range(4):
                n = 4 * dt + g
                lo = 160 + 6 * (n % 4)                       # four rotating sets of six temporaries
                f = [f"v{lo + e}" for e in range(6)]
                for e in range(4):
                    out.append(f"v_accvgpr_read_b32 {f[2 + e]}, a{64 * h + 16 * dt + 4 * g + e}")
                for e in range(4):
                    out.append(f"v_mul_f32_e32 {f[2 + e]}, {f[2 + e]}, {T[7]}")
                if DT == "bf16":
                    out.append(f"v_cvt_pk_bf16_f32 {f[0]}, {f[2]}, {f[3]}")
                    out.append(f"v_cvt_pk_bf16_f32 {f[1]}, {f[4]}, {f[5]}")
                else:
                    for e in range(4):
                        out.append(f"v_cvt_f16_f32_e32 {f[2 + e]}, {f[2 + e]}")
                    out.append(f"v_pack_b32_f16 {f[0]}, {f[2]}, {f[3]}")
                    out.append(f"v_pack_b32_f16 {f[1]}, {f[4]}, {f[5]}")
                out.append(f"ds_write_b64 {WA[n]}, v[{lo}:{lo + 1}]")
        out.append("s_waitcnt lgkmcnt(0)")
        for j in range(8):
            out.append(f"ds_read_b128 {data[j]}, {RB} offset:{1024 * j}")
        for j in range(8):
            # rows 4 j + lane / 16 of the wavefront: stored where the row lies inside the sequence
            out += [f"s_mul_i32 {S_STEP}, %[ostb], {4 * j}",
                    f"v_add_u32_e32 {TMP[j % 2]}, {4 * j}, {RV}",
                    f"v_add_u32_e32 {OFFJ[j % 2]}, {S_STEP}, {SO[j % 4]}",
                    f"v_cmp_gt_u32_e32 vcc, %[olen], {TMP[j % 2]}",
                    f"s_waitcnt lgkmcnt({7 - j})",
                    f"s_and_saveexec_b64 {S_SAVE}, vcc",
                    f"global_store_dwordx4 {OFFJ[j % 2]}, {data[j]}, %[ob{h}] nt",
                    f"s_mov_b64 exec, {S_SAVE}"]
    return out


def program():
    # the common path falls through: top 0, plain body 0, top 1, plain body 1, one branch back
    out = prologue()
    out += select(0) + body(0, False) + select(1) + body(1, False) + ["s_branch .Ltop_0_%="]
    out += [".Lmasked_0_%=:"] + body(0, True) + ["s_branch .Ltop_1_%="]
    out += [".Lmasked_1_%=:"] + body(1, True) + ["s_branch .Ltop_0_%="]
    out += [".Llast_0_%=:"] + body_last(0)
    out += [".Llast_1_%=:"] + body_last(1)
    out += idle_loop()
    out += epilogue()
    return out


HEADER = '''// GENERATED by gen_staircase_pair_core.py -- do not edit; change the generator and regenerate.
//
// Key loop of the staircase attention kernel for a pair of query heads (see the generator's
// docstring for the schedule, the LDS layout and the register map).  Everything between the loads
// of Q and the stores of O happens inside this one asm statement; the physical registers it uses
// are declared as clobbers, the operands are read-only.
@@STRUCT@@__device__ __forceinline__ void @@NAME@@(const PairCoreArgs& A, const @@VEC@@ (&q)[2][8])
{
    asm volatile(
'''


STRUCT = '''struct PairCoreArgs {
    unsigned ka;                     // per-lane LDS byte address of this lane's K fragment of k-step 0 in slot 0
    unsigned val, vah;               // same for the two rows of the V^T fragment of d tile 0
    int jpl;                         // row of the tile whose chunk this lane loads (first of four, 16 apart)
    unsigned ch;                     // byte offset inside a K / V row of the 16-byte chunk this lane loads
    int mrel, mlim;                  // key mask: key visible iff unsigned(key0 + const + mrel) < mlim
    const void* ob0; const void* ob1;  // output of the two heads at the wavefront's first row (which may lie before the sequence)
    unsigned ostb;                   // bytes between consecutive output rows
    unsigned owave;                  // LDS byte address of this wavefront's 8 KB share of a slot
    int orow0, olen;                 // the wavefront's first row relative to the sequence's first token; tokens in the sequence
    const void* kb; const void* vb;  // K / V of this KV head, at the (virtual) row of padded key 0
    unsigned krb, vrb;               // bytes between consecutive K / V rows
    unsigned wrow;                   // LDS byte address of the first row this wavefront loads in slot 0
    int pad, lpm1, nt, whm, whx;     // first valid padded key, last valid padded key, key tiles, first and last key limit of this wavefront
};

'''


def main():
    prog = program()
    text = "\n".join(f'        "{line}\\n"' for line in prog)
    qops = ", ".join(f'[q{h}{ks}] "a"(q[{h}][{ks}])' for h in range(2) for ks in range(8))
    vclob = ", ".join(f'"v{r}"' for r in range(16, 256))
    aclob = ", ".join(f'"a{r}"' for r in list(range(0, 128)) + list(range(192, 224)))
    sclob = ", ".join(f'"s{r}"' for r in range(40, 56))
    tail = f'''
        :
        : [ka] "v"(A.ka), [val] "v"(A.val), [vah] "v"(A.vah), [jpl] "v"(A.jpl), [ch] "v"(A.ch),
          [mrel] "v"(A.mrel), [mlim] "v"(A.mlim),
          [ob0] "s"(A.ob0), [ob1] "s"(A.ob1), [ostb] "s"(A.ostb), [owave] "s"(A.owave), [orow0] "s"(A.orow0), [olen] "s"(A.olen),
          [kb] "s"(A.kb), [vb] "s"(A.vb), [krb] "s"(A.krb), [vrb] "s"(A.vrb), [wrow] "s"(A.wrow),
          [pad] "s"(A.pad), [lpm1] "s"(A.lpm1), [nt] "s"(A.nt), [whm] "s"(A.whm), [whx] "s"(A.whx),
          {qops}
        : "memory", "vcc", "scc", "m0", {sclob},
          {vclob},
          {aclob});
}}
'''
    header = HEADER.replace("@@STRUCT@@", STRUCT if DT == "bf16" else "// (PairCoreArgs: see staircase_pair_core.inc, which is included first)\n\n")
    header = header.replace("@@NAME@@", "staircase_pair_core" if DT == "bf16" else "staircase_pair_core_f16").replace("@@VEC@@", "bf16x8" if DT == "bf16" else "f16x8")
    if DT != "bf16":
        header = header.replace("gen_staircase_pair_core.py --", "gen_staircase_pair_core.py f16 --")
    sys.stdout.write(header + text + tail)
    sys.stderr.write(f"{len(prog)} instructions\n")


if __name__ == "__main__":
    main()
