#!/usr/bin/env python3
"""Writes linear256_loop.inc: the hand-ordered body of linear256_kernel (linear.hip), one string per element type, and the
clobber list of the statement that holds it.

    python3 gen_linear256_loop.py > linear256_loop.inc

The workgroup's four wavefronts own a 256 x 256 output tile, a wavefront 128 x 128 of it as 8 x 8 blocks of 16 x 16
(v_mfma_f32_16x16x32: with random operands the chip sustains 14 % more of these than of the 32x32x16 shape before its
power management lowers the clock).  Block (i, j) = w rows 16i .., x rows 16j .. of the wavefront's part accumulates in
a[4(8i+j) : 4(8i+j)+3]: all 256 AGPRs, which is why the accumulators are not operands of the statement — the text sets
them from the bias, runs the K loop and leaves the converted tile in LDS.

A k-tile is 64 k of both operands in one of two LDS stages (64 KB each: x tile 256 rows x 128 bytes, then the w tile), a
k-step 32 of them: 64 matrix instructions.  Every matrix instruction is followed by at most one LDS operand read (the 16
operands of the next k-step go to the other of two register buffers) and, in a k-tile's second k-step, by at most one
direct global->LDS load of the k-tile after the next.  The one barrier of a k-tile sits behind the first matrix
instruction of its second k-step: by then the wavefront has every operand of this k-tile in registers (its stage may be
overwritten) and its own loads of the next k-tile have landed.

Register plan of a lane (fixed; the kernel names them in the statement's constraints):
    v[56:59]    LDS addresses of the operand reads: 2s = x rows, 2s + 1 = w rows of k-step s (stage bit toggled here)
    v[64:71]    byte offsets of the lane's 8 x-tile loads from the tile's first row      v[72:79]  the same for w
    v[80:87]    LDS addresses of the lane's converted outputs, one per block row i (block column j adds 4096 j)
    v[88:95]    temporaries of the conversion
    v[96:127]   bias of the lane's 32 output columns (4i + e: column 16i + 4(lane/16) + e)
    v[128:191]  operand buffer 0: w blocks 0-7 (4 registers each), then x blocks 0-7      v[192:255]  buffer 1
    s[40:41]    x tile of the next load (advanced here)          s[42:43]  the same for w
    s44  LDS address of the wavefront's first x row in the stage the next loads go to (toggled here)
    s45  k-tiles left        s46  pointer advances left (the loads behind the last k-tile fetch it again: harmless)
"""

RADDR, XOFF, WOFF, EADDR, TMPV, BIAS, BUF0, BUF1 = 56, 64, 72, 80, 88, 96, 128, 192
XPTR, WPTR, M0BASE, LEFT, ADV, TMP = 40, 42, 44, 45, 46, 47
XTILE = 32768


def vr(lo, n=1):
    return "v%d" % lo if n == 1 else "v[%d:%d]" % (lo, lo + n - 1)


def ar(lo, n=1):
    return "a%d" % lo if n == 1 else "a[%d:%d]" % (lo, lo + n - 1)


def frag_reg(buf, kind, blk):
    """kind 0: w block (A operand), 1: x block (B operand)."""
    return (BUF1 if buf else BUF0) + 32 * kind + 4 * blk


# order in which the 16 operands of a k-step are requested: w0, x0 .. x7, w1 .. w7 (matrix instruction n = 8i + j uses w_i, x_j)
READ_ORDER = [(0, 0)] + [(1, j) for j in range(8)] + [(0, i) for i in range(1, 8)]


def first_use(n):
    """Index in READ_ORDER of the last operand matrix instruction n is the first to need, or None."""
    if n == 0:
        return 1
    if n < 8:
        return n + 1
    if n % 8 == 0:
        return 8 + n // 8
    return None


def read(buf, s, q):
    kind, blk = READ_ORDER[q]
    addr = RADDR + 2 * s + (0 if kind == 1 else 1)
    off = 2048 * blk + (XTILE if kind == 0 else 0)
    return "ds_read_b128 %s, %s offset:%d" % (vr(frag_reg(buf, kind, blk), 4), vr(addr), off)


def toggle(s):
    return ["v_xor_b32 %s, 0x10000, %s" % (vr(RADDR + 2 * s), vr(RADDR + 2 * s)),
            "v_xor_b32 %s, 0x10000, %s" % (vr(RADDR + 2 * s + 1), vr(RADDR + 2 * s + 1))]


def dma(i):
    """Load instruction i (0-7: x rows, 8-15: w rows) of the wavefront's share of a k-tile."""
    if i < 8:
        return ["s_add_u32 m0, s%d, %d" % (M0BASE, 1024 * i),
                "global_load_lds_dwordx4 %s, s[%d:%d]" % (vr(XOFF + i), XPTR, XPTR + 1)]
    return ["s_add_u32 m0, s%d, %d" % (M0BASE, XTILE + 1024 * (i - 8)),
            "global_load_lds_dwordx4 %s, s[%d:%d]" % (vr(WOFF + i - 8), WPTR, WPTR + 1)]


def kstep(s, elem):
    mfma = "v_mfma_f32_16x16x32_%s" % elem
    cur, nxt = s, 1 - s
    last = s == 1
    out = []
    issued = 0  # operand reads of the next k-step requested so far
    ndma = 0
    for n in range(64):
        i, j = n >> 3, n & 7
        if last and n == 0:
            out.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
        elif not last and first_use(n) is not None:
            out.append("s_waitcnt lgkmcnt(%d)" % min(15, 15 - first_use(n) + issued))
        load = None
        if last and n >= 2 and (n - 2) % 3 == 0 and ndma < 16:  # m0 a matrix instruction ahead of the load that uses it
            m0, load = dma(ndma)
            out.append(m0)
            ndma += 1
        c = ar(4 * n, 4)
        out.append("%s %s, %s, %s, %s" % (mfma, c, vr(frag_reg(cur, 0, i), 4), vr(frag_reg(cur, 1, j), 4), c))
        if last and n == 0:
            out.append("s_barrier")
        if issued < 16 and n >= (1 if last else 0):
            out.append(read(nxt, 1 - s, issued))
            issued += 1
            if issued == 16:
                out += toggle(1 - s)
        if load:
            out.append(load)
    assert issued == 16 and (ndma == 16 or not last)
    return out


def epilogue(elem):
    """Accumulators -> element type -> the wavefront's quarter of LDS (8 bytes per block and lane)."""
    out = []
    t = TMPV
    for i in range(8):
        for j in range(8):
            a = 4 * (8 * i + j)
            p = t + 4 + 2 * (j & 1)  # alternate the packed pair so that a write's data is not overwritten too early
            for e in range(4):
                out.append("v_accvgpr_read_b32 %s, %s" % (vr(t + e), ar(a + e)))
            if elem == "bf16":
                out.append("v_cvt_pk_bf16_f32 %s, %s, %s" % (vr(p), vr(t), vr(t + 1)))
                out.append("v_cvt_pk_bf16_f32 %s, %s, %s" % (vr(p + 1), vr(t + 2), vr(t + 3)))
            else:
                for e in range(4):
                    out.append("v_cvt_f16_f32 %s, %s" % (vr(t + e), vr(t + e)))
                out.append("v_pack_b32_f16 %s, %s, %s" % (vr(p), vr(t), vr(t + 1)))
                out.append("v_pack_b32_f16 %s, %s, %s" % (vr(p + 1), vr(t + 2), vr(t + 3)))
            out.append("ds_write_b64 %s, %s offset:%d" % (vr(EADDR + i), vr(p, 2), 4096 * j))
    return out


def body(elem):
    out = []
    for i in range(8):
        for j in range(8):
            for e in range(4):
                out.append("v_accvgpr_write_b32 %s, %s" % (ar(4 * (8 * i + j) + e), vr(BIAS + 4 * i + e)))
    for q in range(16):
        out.append(read(0, 0, q))
    out += toggle(0)
    out.append("1:")
    for s in range(2):
        out += kstep(s, elem)
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
            "s_barrier",  # every wavefront has taken its last operands: the stages become the output's staging area
            "s_nop 15", "s_nop 15"]  # (the last matrix instructions' results are read next)
    out += epilogue(elem)
    out.append("s_waitcnt lgkmcnt(0)")
    return out


def main():
    print("// Generated by gen_linear256_loop.py; do not edit.  The body of linear256_kernel: TT_LIN256_BODY_<elem>, and the")
    print("// registers it uses beyond the statement's operands: TT_LIN256_CLOBBERS.")
    print()
    for elem in ("bf16", "f16"):
        print("#define TT_LIN256_BODY_%s \\" % elem.upper())
        print(" \\\n".join('  "%s\\n\\t"' % l for l in body(elem)))
        print()
    regs = ["a%d" % k for k in range(256)] + ["v%d" % k for k in range(TMPV, TMPV + 8)] + ["v%d" % k for k in range(BUF0, 256)]
    regs += ["s%d" % TMP, "m0", "scc", "memory"]
    print("#define TT_LIN256_CLOBBERS \\")
    lines = []
    for k in range(0, len(regs), 16):
        lines.append("  " + ", ".join('"%s"' % r for r in regs[k:k + 16]))
    print(", \\\n".join(lines))
    print()


if __name__ == "__main__":
    main()
