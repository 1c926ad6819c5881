#!/usr/bin/env python3
"""Writes linear256_loop.inc: the hand-ordered K loop of linear256_kernel (linear.hip), one string per element type.

    python3 gen_linear256_loop.py > linear256_loop.inc

The workgroup's four wavefronts own a 256 x 256 output tile, a wavefront 128 x 128 of it as 4 x 4 blocks of 32 x 32 whose
accumulators are the statement's operands c0 .. c15 (block (i, j) = c[4i + j], kept in AGPRs).  A k-tile is 64 k of both
operands in one of two LDS stages (64 KB each: x tile 256 rows x 128 bytes, then the w tile), a k-step 16 of them: 16 matrix
instructions.  The loop is one instruction stream per k-tile in which every matrix instruction is followed by at most
one LDS operand read (the 8 operands of the next k-step go to the other of two register buffers) and, in the last k-step,
by one direct global->LDS load of the k-tile after the next.  The one barrier of a k-tile sits behind the first matrix
instruction of its last k-step: by then the wavefront has every operand of this k-tile in registers (its stage may be
overwritten) and its own loads of the next k-tile have landed.

Register plan of a lane (fixed; the kernel names them in the statement's constraints):
    v[160:167]  byte offsets of the lane's 8 x-tile loads from the tile's first row      v[168:175]  the same for w
    v[176:183]  LDS addresses of the operand reads: 2*ks = x rows, 2*ks + 1 = w rows of k-step ks (stage bit toggled here)
    v[192:223]  operand buffer 0: w blocks 0-3 (4 registers each), then x blocks 0-3      v[224:255]  buffer 1
    s[40:41]    x tile of the next load (advanced here)          s[42:43]  the same for w
    s44  LDS address of the wavefront's first x row in the stage the next loads go to (toggled here)
    s45  k-tiles left        s46  pointer advances left (the loads behind the last k-tile fetch it again: harmless)
"""

XOFF, WOFF, RADDR, BUF0, BUF1 = 160, 168, 176, 192, 224
XPTR, WPTR, M0BASE, LEFT, ADV, TMP = 40, 42, 44, 45, 46, 47
XTILE, STAGE = 32768, 65536


def vr(lo, n=1):
    return "v%d" % lo if n == 1 else "v[%d:%d]" % (lo, lo + n - 1)


def frag_reg(buf, kind, blk):
    """kind 0: w block (A operand), 1: x block (B operand)."""
    return (BUF1 if buf else BUF0) + 16 * kind + 4 * blk


# order in which the operands of a k-step are requested, and the matrix instruction (0-15) that first needs each
READ_ORDER = [(0, 0), (1, 0), (1, 1), (1, 2), (1, 3), (0, 1), (0, 2), (0, 3)]
FIRST_USE = {0: 1, 1: 2, 2: 3, 3: 4, 4: 5, 8: 6, 12: 7}  # matrix instruction -> index in READ_ORDER it waits for


def read(buf, ks, q):
    kind, blk = READ_ORDER[q]
    addr = RADDR + 2 * ks + (0 if kind == 1 else 1)
    off = 4096 * blk + (XTILE if kind == 0 else 0)
    return "ds_read_b128 %s, %s offset:%d" % (vr(frag_reg(buf, kind, blk), 4), vr(addr), off)


def toggle(ks):
    return ["v_xor_b32 %s, 0x10000, %s" % (vr(RADDR + 2 * ks), vr(RADDR + 2 * ks)),
            "v_xor_b32 %s, 0x10000, %s" % (vr(RADDR + 2 * ks + 1), vr(RADDR + 2 * ks + 1))]


def dma(i):
    """Load instruction i (0-7: x rows, 8-15: w rows) of the wavefront's share of a k-tile."""
    if i < 8:
        return ["s_add_u32 m0, s%d, %d" % (M0BASE, 1024 * i),
                "global_load_lds_dwordx4 %s, s[%d:%d]" % (vr(XOFF + i), XPTR, XPTR + 1)]
    return ["s_add_u32 m0, s%d, %d" % (M0BASE, XTILE + 1024 * (i - 8)),
            "global_load_lds_dwordx4 %s, s[%d:%d]" % (vr(WOFF + i - 8), WPTR, WPTR + 1)]


def kstep(ks, elem):
    mfma = "v_mfma_f32_32x32x16_%s" % elem
    cur, nxt = ks & 1, (ks + 1) & 1
    last = ks == 3
    out = []
    issued = 0  # operand reads of the next k-step requested so far
    ndma = 0
    for n in range(16):
        i, j = n >> 2, n & 3
        if last and n == 0:
            out.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
        elif not last and n in FIRST_USE:
            out.append("s_waitcnt lgkmcnt(%d)" % (7 - FIRST_USE[n] + issued))
        if last and 1 <= n and ndma < 16:  # m0 a matrix instruction ahead of the load that uses it
            m0, ld = dma(ndma)
            out.append(m0)
        out.append("%s %%[c%d], %s, %s, %%[c%d]" % (mfma, 4 * i + j, vr(frag_reg(cur, 0, i), 4), vr(frag_reg(cur, 1, j), 4), 4 * i + j))
        if last and n == 0:
            out.append("s_barrier")
        if (last and 1 <= n <= 8) or (not last and n < 8):
            out.append(read(nxt, (ks + 1) & 3, issued))
            issued += 1
            if issued == 8:
                out += toggle((ks + 1) & 3)
        if last and 1 <= n and ndma < 16:
            out.append(ld)
            ndma += 1
            if n == 15:  # sixteen loads in fifteen places
                m0, ld = dma(ndma)
                out += [m0, "s_nop 0", ld]
                ndma += 1
    return out


def loop(elem):
    out = []
    for q in range(8):
        out.append(read(0, 0, q))
    out += toggle(0)
    out.append("1:")
    for ks in range(4):
        out += kstep(ks, elem)
    # the next loads go to the other stage and, while k-tiles are left, to the next k-tile
    out += ["s_xor_b32 s%d, s%d, 0x10000" % (M0BASE, M0BASE),
            "s_cmp_lg_u32 s%d, 0" % ADV,
            "s_cselect_b32 s%d, 128, 0" % TMP,
            "s_add_u32 s%d, s%d, s%d" % (XPTR, XPTR, TMP),
            "s_addc_u32 s%d, s%d, 0" % (XPTR + 1, XPTR + 1),
            "s_add_u32 s%d, s%d, s%d" % (WPTR, WPTR, TMP),
            "s_addc_u32 s%d, s%d, 0" % (WPTR + 1, WPTR + 1),
            "s_lshr_b32 s%d, s%d, 7" % (TMP, TMP),
            "s_sub_u32 s%d, s%d, s%d" % (ADV, ADV, TMP),
            "s_sub_u32 s%d, s%d, 1" % (LEFT, LEFT),
            "s_cmp_lg_u32 s%d, 0" % LEFT,
            "s_cbranch_scc1 1b",
            "s_waitcnt vmcnt(0) lgkmcnt(0)",
            "s_nop 15", "s_nop 15"]  # the last matrix instructions' results are read by ordinary code next
    return out


def main():
    print("// Generated by gen_linear256_loop.py; do not edit.  The K loop of linear256_kernel: TT_LIN256_LOOP_<elem>.")
    print()
    for elem in ("bf16", "f16"):
        print("#define TT_LIN256_LOOP_%s \\" % elem.upper())
        print(" \\\n".join('  "%s\\n\\t"' % l for l in loop(elem)))
        print()


if __name__ == "__main__":
    main()
