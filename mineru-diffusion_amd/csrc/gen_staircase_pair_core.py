#!/usr/bin/env python3
"""Generator of staircase_pair_core.inc: the hand-scheduled gfx950 key loop of the staircase
block-prefill attention kernel for a PAIR of query heads that share a KV head.

Run  python gen_staircase_pair_core.py > staircase_pair_core.inc  after changing the schedule; the
.inc file is what the build compiles.

Why assembly: one wavefront per SIMD has to keep the MFMA pipe busy by itself, so LDS fragment reads
must run several fragments ahead of the MFMA that consumes them and the softmax arithmetic of tile t
has to be issued in the shadow of the MFMAs of tile t+1.  Both need exact control of instruction
order and of physical registers that persist across loop iterations, which neither the compiler's
scheduler nor inline-asm operands (no sub-register access to a 16-register tuple) offer.

Work of one wavefront: 32 query rows x 2 heads, keys in tiles of 64.
  S^T[key, q] = K . Q^T   A = K fragment (LDS, ds_read_b128), B = Q^T (accumulation registers)
  O^T[d, q]  += V^T . P^T A = V^T fragment (LDS, two ds_read_b64_tr_b16), B = P^T (registers)
Every K / V^T fragment feeds the MFMAs of both heads.  Register and key maps are those of
attn_tile.h (key_of_reg, key_of_mfma_row, 272-byte LDS row pitch).

Loop iteration t (S is double-buffered, cb = t & 1):
  X: 32 MFMAs of QK(t+1) -> S[1-cb]   ||  rescale check(t), softmax(t): S[cb] -> P (in place),
     tile t+2: staging registers -> LDS, global loads of tile t+3 -> staging registers
  Y: 32 MFMAs of PV(t)  (P, V slot t) ||  row sums of P(t), row max of S[1-cb], load offsets of tile t+4
  barrier
LDS: three slots each for K and V tiles (slot = tile % 3).

Physical registers (all clobbered; the compiler keeps v0..v39 and a128..a255 for the operands):
  v40..v63   state and temporaries      v64..v191  S[2][head][sub-tile][16]
  v192..v223 staging (K, V: 4 x 16 B)   v224..v247 fragment ring (6 x 4)    v248..v255 temporaries
  a0..a127   O^T[head][d tile][16]      s40..s55   loop state
"""
import sys

PITCH = 272
TILE_BYTES = 64 * PITCH            # 17408
V_RING = 3 * TILE_BYTES            # V slots follow the three K slots
RING_DEPTH = 5                     # fragments in flight
NEG_INF = "v45"                    # holds -inf (a literal would be a second constant-bus read next to vcc)

# ---- register names ---------------------------------------------------------------------------
VPAD, VLPM1, KA, VA, LDSW = "v40", "v41", "v42", "v43", "v44"
ACC = ["v45", "v46", "v47"]                      # spare temporaries
OK = [f"v{48 + p}" for p in range(4)]            # global byte offsets of the next K rows to load
OV = [f"v{52 + p}" for p in range(4)]
M = ["v56", "v57"]
L = ["v58", "v59"]
MX = ["v60", "v61"]
MREL, JP = "v62", "v63"
T = [f"v{248 + i}" for i in range(8)]
S_T, S_KEY0, S_R0, S_R1, S_R2, S_TMP = "s40", "s41", "s42", "s43", "s44", "s45"
S_SAVE = "s[46:47]"


def sreg(b, h, u, i):
    return 64 + 64 * b + 32 * h + 16 * u + i


def stup(b, h, u):
    r = sreg(b, h, u, 0)
    return f"v[{r}:{r + 15}]"


def ptup(b, h, u, t):
    r = sreg(b, h, u, 8 * t)
    return f"v[{r}:{r + 3}]"


def otup(h, dt):
    r = 64 * h + 16 * dt
    return f"a[{r}:{r + 15}]"


def ring(i):
    r = 224 + 4 * (i % 6)
    return f"v[{r}:{r + 3}]", f"v[{r}:{r + 1}]", f"v[{r + 2}:{r + 3}]"


def stg(kv, p):
    r = 192 + 16 * kv + 4 * p
    return f"v[{r}:{r + 3}]"


class Lds:
    """Tracks LDS operations in flight so that waits can be written as exact lgkmcnt values."""

    def __init__(self):
        self.issued = 0

    def op(self, out, text):
        out.append(text)
        self.issued += 1
        return self.issued - 1

    def wait(self, out, idx):
        n = self.issued - 1 - idx
        assert 0 <= n <= 15, n
        out.append(f"s_waitcnt lgkmcnt({n})")

    def drain(self, out):
        out.append("s_waitcnt lgkmcnt(0)")
        self.issued = 0


# ---- VALU fragments -----------------------------------------------------------------------------
def key_const(u, i):
    return 32 * u + 16 * (i >> 3) + 4 * (i & 3) + ((i >> 2) & 1)


def softmax_ops(cb, masked):
    """S[cb] -> P in place, both heads.  Chunks of 8 values; the conversion of a chunk is issued
    one chunk after its exponentials (v_exp results need a gap before a non-transcendental use)."""
    ops = []
    chunks = [(h, u, t) for u in range(2) for t in range(2) for h in range(2)]   # PV consumes (u, t) in this order
    pending = None
    for (h, u, t) in chunks:
        regs = [sreg(cb, h, u, 8 * t + j) for j in range(8)]
        if masked:
            for j, r in enumerate(regs):
                ops.append(f"v_add_u32_e32 {T[j % 4]}, {key_const(u, 8 * t + j)}, {MREL}")
                ops.append(f"v_cmp_lt_u32_e32 vcc, {T[j % 4]}, %[mlim]")
                ops.append(f"v_cndmask_b32_e32 v{r}, {NEG_INF}, v{r}, vcc")
        for r in regs:
            ops.append(f"v_fma_f32 v{r}, v{r}, %[c], -{M[h]}")
        for r in regs:
            ops.append(f"v_exp_f32_e32 v{r}, v{r}")
        if pending:
            ops += pending
        base = sreg(cb, h, u, 8 * t)
        pending = [f"v_cvt_pk_bf16_f32 v{base + j}, v{base + 2 * j}, v{base + 2 * j + 1}" for j in range(4)]
    ops.append("s_nop 0")
    ops += pending
    return ops


def rowsum_ops(cb):
    """l[h] += sum of the bf16 probabilities of tile t (two accumulation chains per head)."""
    ops = []
    part = {0: (L[0], T[4]), 1: (L[1], T[5])}
    ops.append(f"v_mov_b32_e32 {T[4]}, 0")
    ops.append(f"v_mov_b32_e32 {T[5]}, 0")
    k = 0
    for u in range(2):
        for t in range(2):
            for j in range(4):
                for h in range(2):
                    r = sreg(cb, h, u, 8 * t + j)
                    acc = part[h][k & 1]
                    ops.append(f"v_dot2_f32_bf16 {acc}, v{r}, %[ones], {acc}")
                k += 1
    ops.append("s_nop 3")        # a dot result needs 3 wait states before a VALU of another kind reads it
    for h in range(2):
        ops.append(f"v_add_f32_e32 {L[h]}, {L[h]}, {part[h][1]}")
    return ops


def rowmax_ops(b):
    """MX[h] = max over this query's 64 keys of S[b][h] (raw scores, both half-waves)."""
    ops = []
    for h in range(2):
        regs = [sreg(b, h, u, i) for u in range(2) for i in range(16)]
        a, c = T[2 * h], T[2 * h + 1]
        ops.append(f"v_max3_f32 {a}, v{regs[0]}, v{regs[1]}, v{regs[2]}")
        ops.append(f"v_max3_f32 {c}, v{regs[3]}, v{regs[4]}, v{regs[5]}")
        rest = regs[6:]                              # 26 values, two per further step, alternating chains
        for i in range(0, len(rest), 2):
            d = a if (i >> 1) % 2 == 0 else c
            ops.append(f"v_max3_f32 {d}, {d}, v{rest[i]}, v{rest[i + 1]}")
        ops.append(f"v_max_f32_e32 {a}, {a}, {c}")
    for h in range(2):
        a, c = T[2 * h], T[2 * h + 1]
        ops.append(f"v_mov_b32_e32 {c}, {a}")
    ops.append("s_nop 1")
    for h in range(2):
        a, c = T[2 * h], T[2 * h + 1]
        ops.append(f"v_permlane32_swap_b32_e32 {a}, {c}")
    ops.append("s_nop 1")
    for h in range(2):
        a, c = T[2 * h], T[2 * h + 1]
        ops.append(f"v_max_f32_e32 {MX[h]}, {a}, {c}")
    return ops


def load_offset_ops():
    """Byte offsets of the rows the next global loads fetch (rows clamped into the sequence), then JP += 64."""
    ops = []
    for p in range(4):
        ops.append(f"v_add_u32_e32 {T[6]}, {16 * p}, {JP}")
        ops.append(f"v_med3_i32 {T[6]}, {T[6]}, {VPAD}, {VLPM1}")
        ops.append(f"v_mul_lo_u32 {OK[p]}, {T[6]}, %[krb]")
        ops.append(f"v_mul_lo_u32 {OV[p]}, {T[6]}, %[vrb]")
        ops.append(f"v_add_u32_e32 {OK[p]}, {OK[p]}, %[ck]")
        ops.append(f"v_add_u32_e32 {OV[p]}, {OV[p]}, %[ck]")
    ops.append(f"v_add_u32_e32 {JP}, 64, {JP}")
    return ops


def global_loads():
    out = []
    for p in range(4):
        out.append(f"global_load_dwordx4 {stg(0, p)}, {OK[p]}, %[kb]")
        out.append(f"global_load_dwordx4 {stg(1, p)}, {OV[p]}, %[vb]")
    return out


def stage_writes(lds, out, slot_sreg):
    """Staging registers -> LDS slot whose byte offset is in slot_sreg."""
    out.append("s_waitcnt vmcnt(0)")
    out.append(f"v_add_u32_e32 {LDSW}, {slot_sreg}, %[ldswr]")
    for p in range(4):
        lds.op(out, f"ds_write_b128 {LDSW}, {stg(0, p)} offset:{4352 * p}")
        lds.op(out, f"ds_write_b128 {LDSW}, {stg(1, p)} offset:{V_RING + 4352 * p}")


def check_rescale(uid):
    """Running-max update of both heads from MX (lazy: only when some query exceeds the stale max
    by more than 2^8); the rare path rescales l and O^T (accumulation registers) in place."""
    out = []
    for h in range(2):
        lab = f".Lskip_{uid}_{h}_%="
        out.append(f"v_mul_f32_e32 {T[0]}, %[c], {MX[h]}")
        out.append(f"v_max_f32_e32 {T[0]}, {T[0]}, {M[h]}")
        out.append(f"v_add_f32_e32 {T[1]}, 0x41000000, {M[h]}")
        out.append(f"v_cmp_gt_f32_e32 vcc, {T[0]}, {T[1]}")
        out.append(f"s_cbranch_vccz {lab}")
        out.append(f"v_sub_f32_e32 {T[1]}, {M[h]}, {T[0]}")
        out.append(f"v_exp_f32_e32 {T[1]}, {T[1]}")
        out.append(f"v_mov_b32_e32 {M[h]}, {T[0]}")
        out.append("s_nop 15")                      # the MFMAs of the previous tile's PV have long finished; margin only
        out.append(f"v_mul_f32_e32 {L[h]}, {L[h]}, {T[1]}")
        for i in range(64):
            a = f"a{64 * h + i}"
            t = T[2 + (i & 3)]
            out.append(f"v_accvgpr_read_b32 {t}, {a}")
            out.append(f"v_mul_f32_e32 {t}, {t}, {T[1]}")
            out.append(f"v_accvgpr_write_b32 {a}, {t}")
        out.append("s_nop 7")
        out.append(f"{lab}:")
    return out


# ---- MFMA streams -------------------------------------------------------------------------------
def qk_stream(nb):
    """[(reads, mfmas)] per K fragment n: fragment (u = n & 1, ks = n >> 1) -> S[nb][h][u] for h = 0, 1."""
    items = []
    for n in range(16):
        u, ks = n & 1, n >> 1
        frag = ring(n)[0]
        rd = [f"ds_read_b128 {frag}, {KA} offset:{u * 32 * PITCH + ks * 32}"]
        mf = []
        for h in range(2):
            c = "0" if ks == 0 else stup(nb, h, u)
            mf.append(f"v_mfma_f32_32x32x16_bf16 {stup(nb, h, u)}, {frag}, %[q{h}{ks}], {c}")
        items.append((rd, mf))
    return items


def pv_stream(cb):
    """Fragment m: (u, t, dt) = (m >> 3, (m >> 2) & 1, m & 3); O^T[h][dt] += V^T frag . P[h][u][t]."""
    items = []
    for m in range(16):
        u, t, dt = m >> 3, (m >> 2) & 1, m & 3
        frag, lo, hi = ring(m)
        o = (u * 32 + t * 16) * PITCH + dt * 64
        rd = [f"ds_read_b64_tr_b16 {lo}, {VA} offset:{o}", f"ds_read_b64_tr_b16 {hi}, {VA} offset:{o + PITCH}"]
        mf = [f"v_mfma_f32_32x32x16_bf16 {otup(h, dt)}, {frag}, {ptup(cb, h, u, t)}, {otup(h, dt)}" for h in range(2)]
        items.append((rd, mf))
    return items


def interleave(out, lds, items, valu, extras=None):
    """MFMA stream with a read-ahead of RING_DEPTH fragments; VALU ops are dealt evenly into the
    slots after each MFMA; extras = {fragment index: [instructions or callables]} are placed after
    that fragment's MFMAs."""
    extras = extras or {}
    n_slots = 2 * len(items)
    per = [len(valu) // n_slots + (1 if i < len(valu) % n_slots else 0) for i in range(n_slots)]
    vi = 0
    ids = {}
    for n in range(min(RING_DEPTH, len(items))):
        for r in items[n][0]:
            ids[n] = lds.op(out, r)
    slot = 0
    for n, (rd, mf) in enumerate(items):
        lds.wait(out, ids[n])
        for mi, mfma in enumerate(mf):
            out.append(mfma)
            for _ in range(per[slot]):
                out.append(valu[vi])
                vi += 1
            slot += 1
        nxt = n + RING_DEPTH
        if nxt < len(items):
            for r in items[nxt][0]:
                ids[nxt] = lds.op(out, r)
        for e in extras.get(n, []):
            if callable(e):
                e(out)
            else:
                out.append(e)
    assert vi == len(valu)


# ---- program ------------------------------------------------------------------------------------
def prologue():
    out = []
    lds = Lds()
    out += [f"v_mov_b32_e32 {NEG_INF}, 0xff800000", f"v_mov_b32_e32 {VPAD}, %[pad]", f"v_mov_b32_e32 {VLPM1}, %[lpm1]",
            f"v_mov_b32_e32 {MREL}, %[mrel]", f"v_mov_b32_e32 {JP}, %[jp0]"]
    for h in range(2):
        out += [f"v_mov_b32_e32 {M[h]}, 0xf149f2ca", f"v_mov_b32_e32 {L[h]}, 0"]      # -1e30
    for i in range(128):
        out.append(f"v_accvgpr_write_b32 a{i}, 0")
    out += [f"s_mov_b32 {S_T}, 0", f"s_mov_b32 {S_KEY0}, 0", f"s_mov_b32 {S_R0}, 0",
            f"s_mov_b32 {S_R1}, {TILE_BYTES}", f"s_mov_b32 {S_R2}, {2 * TILE_BYTES}"]
    # tiles 0 and 1 -> LDS slots 0 and 1; tile 2 -> staging registers; offsets of tile 3 prepared
    for slot in (S_R0, S_R1):
        out += load_offset_ops()
        out += global_loads()
        stage_writes(lds, out, slot)
    out += load_offset_ops()
    out += global_loads()
    out += load_offset_ops()
    lds.drain(out)
    out.append("s_barrier")
    # QK(0) -> S[0], row max of tile 0
    out.append(f"v_add_u32_e32 {KA}, {S_R0}, %[ka]")
    interleave(out, lds, qk_stream(0), [])
    out.append("s_nop 15")
    out += rowmax_ops(0)
    return out


def body(cb, masked):
    uid = f"{cb}{int(masked)}"
    out = []
    lds = Lds()
    nb = 1 - cb
    out += check_rescale(uid)
    # ---- X
    out.append(f"v_add_u32_e32 {KA}, {S_R1}, %[ka]")
    extras = {1: [lambda o: stage_writes(lds, o, S_R2)], 7: global_loads()}
    interleave(out, lds, qk_stream(nb), softmax_ops(cb, masked), extras)
    out.append("s_nop 1")
    # ---- Y
    out.append(f"v_add_u32_e32 {VA}, {S_R0}, %[va]")
    yv = rowsum_ops(cb)
    pre = ["s_nop 7"]                       # S[nb] was written by the last MFMAs of X
    yv_late = rowmax_ops(nb) + load_offset_ops()
    items = pv_stream(cb)
    # row max may only start once the QK MFMAs have retired: give the sums the first slots
    interleave(out, lds, items, yv + pre + yv_late)
    lds.drain(out)
    # ---- loop state
    out += [f"s_mov_b32 {S_TMP}, {S_R0}", f"s_mov_b32 {S_R0}, {S_R1}", f"s_mov_b32 {S_R1}, {S_R2}", f"s_mov_b32 {S_R2}, {S_TMP}",
            f"s_add_i32 {S_T}, {S_T}, 1", f"s_add_i32 {S_KEY0}, {S_KEY0}, 64", f"v_add_u32_e32 {MREL}, 64, {MREL}",
            "s_barrier"]
    return out


def dispatch(cb):
    """Chooses the masked or the plain body for tile t (wavefront-uniform)."""
    out = [f".Ltop_{cb}_%=:",
           f"s_cmp_ge_i32 {S_T}, %[nt]",
           "s_cbranch_scc1 .Lend_%=",
           f"s_cmp_lt_i32 {S_KEY0}, %[pad]",
           f"s_cbranch_scc1 .Lbody_{cb}1_%=",
           f"s_add_i32 {S_TMP}, {S_KEY0}, 64",
           f"s_cmp_gt_i32 {S_TMP}, %[whm]",
           f"s_cbranch_scc1 .Lbody_{cb}1_%="]
    for masked in (False, True):
        out.append(f".Lbody_{cb}{int(masked)}_%=:")
        out += body(cb, masked)
        out.append(f"s_branch .Ltop_{1 - cb}_%=")
    return out


def epilogue():
    out = [".Lend_%=:", "s_nop 15", "s_nop 15"]
    out += [f"v_cmp_ne_u32_e32 vcc, 0, %[ok]", f"s_and_saveexec_b64 {S_SAVE}, vcc"]
    for h in range(2):
        out += [f"v_mov_b32_e32 {T[7]}, {L[h]}", "s_nop 1", f"v_permlane32_swap_b32_e32 {L[h]}, {T[7]}", "s_nop 1",
                f"v_add_f32_e32 {T[7]}, {L[h]}, {T[7]}", f"v_rcp_f32_e32 {T[7]}, {T[7]}", "s_nop 0"]
        for dt in range(4):
            for g in range(4):
                for e in range(4):
                    out.append(f"v_accvgpr_read_b32 {T[2 + e]}, a{64 * h + 16 * dt + 4 * g + e}")
                for e in range(4):
                    out.append(f"v_mul_f32_e32 {T[2 + e]}, {T[2 + e]}, {T[7]}")
                out.append(f"v_cvt_pk_bf16_f32 {T[0]}, {T[2]}, {T[3]}")
                out.append(f"v_cvt_pk_bf16_f32 {T[1]}, {T[4]}, {T[5]}")
                out.append(f"global_store_dwordx2 %[o{h}], v[248:249], off offset:{(dt * 32 + 8 * g) * 2}")
    out += [f"s_mov_b64 exec, {S_SAVE}", "s_waitcnt vmcnt(0)"]
    return out


def program():
    out = prologue()
    out.append("s_branch .Ltop_0_%=")
    out += dispatch(0)
    out += dispatch(1)
    out += epilogue()
    return out


HEADER = '''// GENERATED by gen_staircase_pair_core.py -- do not edit; change the generator and regenerate.
//
// Key loop of the staircase attention kernel for a pair of query heads (see the generator's
// docstring for the schedule and the register map).  Everything between the loads of Q and the
// stores of O happens inside this one asm statement; the physical registers it uses are declared
// as clobbers, the operands are read-only.
struct PairCoreArgs {
    unsigned ldswr, ka, va;          // per-lane LDS byte addresses: staging write, K fragment read, V^T fragment read (slot 0)
    int jp0;                         // row of the tile this thread stages (threadIdx / 16)
    unsigned ck;                     // byte offset of this thread's 16-byte chunk inside a row
    int mrel, mlim;                  // key mask: key visible iff unsigned(key0 + const + mrel) < mlim
    __bf16* o0; __bf16* o1;          // output rows of the two heads (+ 4 * half-wave elements)
    int ok;                          // this lane's query row exists
    const void* kb; const void* vb;  // K / V of this KV head, at the (virtual) row of padded key 0
    unsigned krb, vrb;               // bytes between consecutive K / V rows
    int pad, lpm1, nt, whm;          // first valid padded key, last valid padded key, key tiles, first limit of this wavefront
    float c;                         // softmax scale * log2(e)
};

__device__ __forceinline__ void staircase_pair_core(const PairCoreArgs& A, const bf16x8 (&q)[2][8])
{
    asm volatile(
'''


def main():
    prog = program()
    text = "\n".join(f'        "{line}\\n"' for line in prog)
    qops = ", ".join(f'[q{h}{ks}] "a"(q[{h}][{ks}])' for h in range(2) for ks in range(8))
    vclob = ", ".join(f'"v{r}"' for r in range(40, 256))
    aclob = ", ".join(f'"a{r}"' for r in range(0, 128))
    sclob = ", ".join(f'"s{r}"' for r in range(40, 56))
    tail = f'''
        :
        : [ldswr] "v"(A.ldswr), [ka] "v"(A.ka), [va] "v"(A.va), [jp0] "v"(A.jp0), [ck] "v"(A.ck),
          [mrel] "v"(A.mrel), [mlim] "v"(A.mlim), [o0] "v"(A.o0), [o1] "v"(A.o1), [ok] "v"(A.ok),
          [kb] "s"(A.kb), [vb] "s"(A.vb), [krb] "s"(A.krb), [vrb] "s"(A.vrb), [pad] "s"(A.pad), [lpm1] "s"(A.lpm1),
          [nt] "s"(A.nt), [whm] "s"(A.whm), [c] "s"(A.c), [ones] "s"(0x3f803f80u),
          {qops}
        : "memory", "vcc", "scc", {sclob},
          {vclob},
          {aclob});
}}
'''
    sys.stdout.write(HEADER + text + tail)
    sys.stderr.write(f"{len(prog)} instructions\n")


if __name__ == "__main__":
    main()
