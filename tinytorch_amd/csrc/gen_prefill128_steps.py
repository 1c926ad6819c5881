#!/usr/bin/env python3
"""Writes prefill128_steps.inc: the hand-ordered instruction streams of the pipelined prefill kernel's steady state
(sdpa_prefill_d128.hip), one string per (tile of the 4-tile unrolled body, step of the tile, element type).

    python3 gen_prefill128_steps.py > prefill128_steps.inc         (head_dim 128, sdpa_prefill_d128.hip)
    python3 gen_prefill128_steps.py 64 > prefill64_steps.inc       (head_dim 64, sdpa_prefill_d64.hip)

A step is 16 slots, one matrix instruction each (even slot: S^T k-step, odd slot: P.V product), with the vector work
of one score (scale/shift, exp2, running sum, conversion of a pair) spread over the slots so that no instruction
waits for the one before it, and the LDS operand of the slot PD places ahead requested into a ring of 8 operand
registers.  The compiler's own ordering of the same step left the matrix pipe idle a third of the time: a wavefront
issues in order, and a chain fma -> exp2 -> add of one score issued back to back stalls on each result.

Register plan of a lane (fixed, named in the statements' constraints by the kernel):
    v[120:151]  Q operands, 8 k-steps x 4 registers
    v[152:159]  V operand addresses (LDS bytes, the V region's base folded in), index 2*db + ld
    v[160:175]  score accumulator "B"      v[176:191]  score accumulator "C"
    v[192:199]  probabilities "A" (2 k-steps x 4)      v[200:207]  probabilities "B"
    v[208:239]  operand ring, 8 x 4        v[240:247]  temporaries      v[248:255]  K operand addresses, one per k-step
Named operands of the statement: o0-o3 the four output accumulators (read-write), ps the lane's sum of the step's
probabilities (out), c = scale*log2(e) (scalar register), mc = maximum*scale*log2(e), and for the causal variant
mk (scalar, 1 = take it), kvs (scalar, first key of the half whose exponentials the step takes) and rl (query row of
the lane in key coordinates - 4*(lane/32)).

Every string holds the step twice: as above, and with the causal predicate applied to each probability (a score's
key is visible iff kvs + 8*(n/4) + n%4 <= rl: two more instructions per score, a compare through m0 and vcc and a
select).  The second form serves the one or two tiles of a wavefront's row group that touch the diagonal; it sits out
of line, in subsection 1 of the kernel's section, so that the steady state falls through without a taken branch.

Calls with a Bool attnMask have a third form of the plain step, TT_P128_MSTEP_... (TT_P64_MSTEP_...): a score's probability is
kept iff its mask byte is set (a compare on one byte of a register through SDWA and a select: two more instructions per
score).  A lane's 16 mask bytes of a 32-key half are four dwords (keys 8g + 4*(lane/32) .. +3 of the lane's query row, g = 0..3) in
    v[112:119]  mask registers: 2 halves x 4 dwords, half H in place H % 2
The mask bytes of a tile (a wavefront's 32 rows x 64 keys: 2 KiB) come into LDS by direct loads two tiles ahead
(TT_P128_MDMA: 2 loads of 16 whole 64-byte row segments each, 16 bytes per lane, so a tile costs 32 line requests where
loads of every lane's own dwords cost 256) into a ring of two tiles per wavefront: rows 16i .. 16i+15 in KiB i of the
tile, the 16-byte chunk c of a row segment at 256 c + 16 (row % 16).  A step starts by reading the lane's four dwords of
the half after next with two ds_read2_b32 (dwords h and h + 2 of chunks 2H and 2H + 1, h = lane/32, H the half of the tile;
operand mlds: the lane's row in the ring + 4h; TT_P128_MREAD_FIRST: the half the workgroup's first step takes).
"""
import sys

PD, RING = 6, 8
MASK0, Q0, VADDR0, SB0, SC0, PA0, PB0, RING0, T0, KADDR0 = 112, 120, 152, 160, 176, 192, 200, 208, 240, 248
# set by configure(head_dim): k-steps of a score product (= P.V products of a half), head_dim blocks of 32, slots of a
# step, scores whose vector work a slot carries, bytes of a tile row and of a stage, slots of the 4-tile body
KST = NDB = NS = SPS = ROW = STAGE = BODY = 0
NAME = ""


def configure(head_dim):
    global KST, NDB, NS, SPS, ROW, STAGE, BODY, NAME
    KST, NDB = head_dim // 16, head_dim // 32
    NS = 2 * KST
    SPS = 16 // NS
    ROW = 2 * head_dim
    STAGE = 64 * ROW
    BODY = 8 * NS
    NAME = "P%d" % head_dim


def vr(lo, n=1):
    return "v%d" % lo if n == 1 else "v[%d:%d]" % (lo, lo + n - 1)


def fetch(G):
    """LDS operand request of slot G of the 4-tile body into its ring place."""
    G %= BODY
    u, kind, s = G // (2 * NS), (G // NS) % 2, G % NS
    i, r = s >> 1, RING0 + 4 * (G % RING)
    if s % 2 == 0:  # K rows of half `kind` of tile u+1, k-step i
        off = ((u + 1) & 3) * STAGE + kind * 32 * ROW
        return ["ds_read_b128 %s, %s offset:%d" % (vr(r, 4), vr(KADDR0 + i), off)]
    t, db = i // NDB, i % NDB  # V^T of half `kind` of tile u, keys 16t..16t+15, head_dim block db
    off = u * STAGE + kind * 32 * ROW + 16 * t * ROW
    return ["ds_read_b64_tr_b16 %s, %s offset:%d" % (vr(r, 2), vr(VADDR0 + 2 * db), off),
            "ds_read_b64_tr_b16 %s, %s offset:%d" % (vr(r + 2, 2), vr(VADDR0 + 2 * db + 1), off)]


def pending_after(G):
    """LDS requests issued after the operand of slot G and before slot G's matrix instruction."""
    return sum(len(fetch(g)) for g in range(G + 1, G + PD))


def step(u, kind, elem, masked=False, bmask=False):
    mfma = "v_mfma_f32_32x32x16_%s" % elem
    cvt = "v_cvt_pk_%s_f32" % elem
    G0 = 2 * NS * u + NS * kind
    s_new, s_nxt = (SC0, SB0) if kind == 0 else (SB0, SC0)
    p_cur, p_nxt = (PA0, PB0) if kind == 0 else (PB0, PA0)
    F = [T0 + 4, T0 + 5]
    T = [T0, T0 + 1, T0 + 2, T0 + 3]
    out = []
    fma = lambda n: "v_fma_f32 %s, %s, %%[c], -%%[mc]" % (vr(F[n & 1]), vr(s_nxt + n))

    def hide(n):  # causal mask of score n: visible iff kvs + 8*(n/4) + n%4 <= rl (kvs: first key of the half, rl = query - 4*(lane/32))
        return ["s_add_i32 m0, %%[kvs], %d" % (8 * (n >> 2) + (n & 3)), "v_cmp_le_i32 vcc, m0, %[rl]",
                "v_cndmask_b32 %s, 0, %s, vcc" % (vr(T[n & 3]), vr(T[n & 3]))]

    def vector_work(n):  # of score n: its exp2, the next score's scale/shift, the previous score's add, a pair's conversion
        w = ["v_exp_f32 %s, %s" % (vr(T[n & 3]), vr(F[n & 1]))]
        if n + 1 < 16:
            w.append(fma(n + 1))
        if masked:
            w += hide(n)
        if bmask:  # keep the probability iff the score's mask byte is set: byte n%4 of dword n/4 of the half's place
            place = (kind + 1) & 1  # the step takes the exponentials of half 2j + kind + 1
            w += ["v_cmp_ne_u32_sdwa vcc, %s, %%[zero] src0_sel:BYTE_%d src1_sel:DWORD" % (vr(MASK0 + 4 * place + (n >> 2)), n & 3),
                  "v_cndmask_b32 %s, 0, %s, vcc" % (vr(T[n & 3]), vr(T[n & 3]))]
        if n == 2:  # the sum starts as (score 0) + (score 1): what 0 + x0 + x1 gives
            w.append("v_add_f32 %%[ps], %s, %s" % (vr(T[0]), vr(T[1])))
        elif n >= 3:
            w.append("v_add_f32 %%[ps], %%[ps], %s" % vr(T[(n - 1) & 3]))
        if n % 2 == 0 and n >= 2:
            j = (n - 2) // 2  # scores n-2, n-1
            w.append("%s %s, %s, %s" % (cvt, vr(p_nxt + j), vr(T[(n - 2) & 3]), vr(T[(n - 1) & 3])))
        return w

    out.append(fma(0))
    extra = 0
    if bmask:  # the mask dwords of half 2j + kind + 2 (tile j+1, its half `kind`) from the wavefront's ring in LDS
        out += mask_reads((u + 1) & 1, kind, kind & 1)
        extra = 2  # requests behind those of the step's first operands
    for n in range(NS):
        G = G0 + n
        r = RING0 + 4 * (G % RING)
        out.append("s_waitcnt lgkmcnt(%d)" % (pending_after(G) + (extra if n < PD else 0)))
        if n % 2 == 0:
            ks = n // 2
            c = "0" if n == 0 else vr(s_new, 16)
            out.append("%s %s, %s, %s, %s" % (mfma, vr(s_new, 16), vr(r, 4), vr(Q0 + 4 * ks, 4), c))
        else:
            i = n // 2
            out.append("%s %%[o%d], %s, %s, %%[o%d]" % (mfma, i % NDB, vr(r, 4), vr(p_cur + 4 * (i // NDB), 4), i % NDB))
        out += fetch(G + PD)  # directly behind the matrix instruction: measured 0.7% faster than behind the vector work
        for q in range(SPS * n, SPS * (n + 1)):
            out += vector_work(q)
    if not masked:
        out.append("s_nop 0")
    out.append("v_add_f32 %%[ps], %%[ps], %s" % vr(T[15 & 3]))
    out.append("%s %s, %s, %s" % (cvt, vr(p_nxt + 7), vr(T[14 & 3]), vr(T[15 & 3])))
    return out


def prefetch():
    out = []
    for g in range(PD):
        out += fetch(g)
    return out


def mask_reads(region, half, place):
    """The four mask dwords of half `half` of the tile in ring place `region` into register place `place`."""
    if region:  # the second ring place lies beyond the 8-bit dword offsets of ds_read2_b32: its own address operand
        return ["ds_read2_b32 %s, %%[mlds1] offset0:%d offset1:%d" % (vr(MASK0 + 4 * place + 2 * c, 2), 128 * half + 64 * c, 128 * half + 64 * c + 2) for c in range(2)]
    return ["ds_read2_b32 %s, %%[mlds] offset0:%d offset1:%d" % (vr(MASK0 + 4 * place + 2 * c, 2), 128 * half + 64 * c, 128 * half + 64 * c + 2) for c in range(2)]


def mask_dma():
    """A tile's mask bytes into the wavefront's ring in LDS: load i brings the 64-byte segments of rows 16i .. 16i+15
    (operands o0, o1: the lane's byte offset for each — its row, rows past the end moved back, and 16-byte chunk; mtile:
    scalar address of the tile's first key in the mask; dst: LDS address of the ring place).  s_nop 4: the scalar address may
    have been restored by a vector instruction."""
    out = ["s_nop 4"]
    for i in range(2):
        out += ["s_add_u32 m0, %%[dst], %d" % (1024 * i), "s_nop 0", "global_load_lds_dwordx4 %%[o%d], %%[mtile]" % i]
    return out


def emit(name, lines):
    print("#define %s \\" % name)
    print(" \\\n".join('  "%s\\n\\t"' % l for l in lines))
    print()


def main():
    head_dim = 128
    if len(sys.argv) > 1:
        head_dim = int(sys.argv[1])
    configure(head_dim)
    lab = ".Ltt_%s" % NAME.lower()
    print("// Generated by gen_prefill128_steps.py%s; do not edit.  Instruction streams of the pipelined prefill kernel's" % ("" if head_dim == 128 else " %d" % head_dim))
    print("// steady state: TT_%s_STEP_<elem>_U<tile of the unrolled body>_K<step of the tile> (with the causal variant out of" % NAME)
    print("// line), TT_%s_PSTEP_... the plain step alone." % NAME)
    print()
    emit("TT_%s_PREFETCH" % NAME, prefetch())
    for elem in ("bf16", "f16"):
        for u in range(4):
            for kind in range(2):
                # the variant with the causal predicate sits out of line (at the end of the kernel's section), so that the
                # steady state runs through without a taken branch
                both = (["s_cmp_eq_u32 %[mk], 0", "s_cbranch_scc0 %s_m%%=" % lab] + step(u, kind, elem) + ["%s_e%%=:" % lab, ".subsection 1", "%s_m%%=:" % lab]
                        + step(u, kind, elem, True) + ["s_branch %s_e%%=" % lab, ".subsection 0"])
                emit("TT_%s_STEP_%s_U%d_K%d" % (NAME, elem.upper(), u, kind), both)
                emit("TT_%s_PSTEP_%s_U%d_K%d" % (NAME, elem.upper(), u, kind), step(u, kind, elem))  # calls without a causal mask
                emit("TT_%s_MSTEP_%s_U%d_K%d" % (NAME, elem.upper(), u, kind), step(u, kind, elem, bmask=True))  # Bool attnMask
    emit("TT_%s_MDMA" % NAME, mask_dma())
    # before the first step of a workgroup (tile index a multiple of 4: ring place 0): the half it takes, half 1 of that tile
    # (waited for at once: the first tile's own loads go to the same ring place)
    emit("TT_%s_MREAD_FIRST" % NAME, mask_reads(0, 1, 1) + ["s_waitcnt lgkmcnt(0)"])


if __name__ == "__main__":
    main()
