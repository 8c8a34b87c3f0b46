#!/usr/bin/env python3
"""Generates int4wo_gemv1_loop.inc: the software-pipelined tile loop of int4wo_gemv1_kernel as one inline-asm string.

Run `python gen_int4wo_gemv1.py > int4wo_gemv1_loop.inc` after changing the schedule; the generated file is committed
and tests/test_gemv1_codegen.py checks that it is what this script prints and that the schedule keeps the hardware's
dependency distances.

What the loop does (one wave, one 16-row block of the packed weight, a run of 128-wide K tiles)
----------------------------------------------------------------------------------------------
Lane l = 4 * row + i loads the 16-byte chunk (row, k quarter i) of every tile: 32 codes of one row, all in one
quantization group, lanes 0,1 of a 4-lane block in one group and lanes 2,3 in one group (group size >= 64).
Dequantization keeps both bf16 roundings of dequantize_affine, w = bf16(bf16((q - 8) * s) + z), and runs on the
4x4x4 matrix instructions (16 independent 4x4 blocks, one per 4 lanes, two passes):

  X   p  = v_and_b32_dpp(w or w >> 8, mask)   two codes per register as fp16 subnormals q * 2^-24 (lanes 0,1 of a
                                              block, mask 0x000F000F) or q * 2^-20 (lanes 2,3, mask 0x00F000F0);
                                              quad_perm [0,1,0,1] fetches register 0 from the block's lanes 0 / 1,
                                              [2,3,2,3] register 1 from lanes 2 / 3, so position k of a lane's four
                                              codes belongs to the group whose parameters lane k of the block holds
  M1  d  = a1 * p + c1      (f16 4x4x4)       a1 = mantissa m of lane k's scale (s = m * 2^E) at position k,
                                              c1 = -8 m f  (f = 2^-24 or 2^-20): d = (q - 8) m f, exact
  R1  t  = cvt_pk_bf16(d)                     first rounding (exact scaling by f and 2^E commutes with it)
  M2  u  = a2 * t + c2      (bf16 4x4x4)      a2 = 2^E (with the scale's sign) at position k, c2 = z f: u = (T + z) f
  R2  wv = cvt_pk_bf16(u)                     second rounding: the dequantized weight times f
  P   acc += x * wv         (bf16 4x4x4)      A operand = the lane's own four activations; element l % 4 of acc is the
                                              lane's partial dot product, the caller multiplies it by 1 / f

Activations come from LDS, where the caller has laid a tile's 128 values out in the order the lanes consume them:
tile t, step pair sp (two steps = 16 bytes), lane type j = l % 4 at byte 256 t + 64 sp + 16 j; a ds_read_b128 of the
16 lanes of a row group then covers 64 contiguous bytes.

One step per four codes; stage s of quad u runs in step u + s so that every matrix result is read five or more issue
slots after its instruction and every VALU result two or more slots before a matrix instruction or a DPP read.
The per-tile parameters (a1, a2, c1, c2) of the next tile are built one instruction per step (7 VALU + 2 matrix).
Weight tiles stream through a ring of D register buffers filled by global_load ... nt; a run of up to D tiles is
requested whole before its first tile is touched.  A tile's body waits for the NEXT tile only in its last step, with
the exact count of younger requests; once the run's last tile has been requested the loop stops requesting (a
repeated request would be served by memory again).  The (scale, zero) words come from LDS too, 128 bytes per tile in the order
[k half][row], staged by the caller.

`python gen_int4wo_gemv1.py --v2 > int4wo_gemv2_loop.inc` prints the variant for int4wo_gemv2_kernel (one 16-wave
workgroup per CU): a wave's run is a contiguous piece of the workgroup's tile stream and may cross unit boundaries
(a unit = the K range of one row block, or one of its equal parts when K is split).  Differences:
  * the activation row sits ONCE in the workgroup's LDS, 256 bytes per K tile; the loop keeps the address of the current
    and of the next tile (xa, xn) and wraps the tile index at the end of a row block (scalars ktn, kbx);
  * at a unit boundary, and after the last tile, the accumulator is reduced over the four lanes of a row exactly as the
    kernel's epilogue does (own element, times 1 / f, two quad-permute adds) and stored to the wave's next 256-byte
    slot of partial sums in LDS (every lane stores; the four lanes of a row hold the same sum); the block has no
    register output.  The flush of a finished unit runs in step 3 of the next tile, after that unit's last product.
"""
import sys

V2 = "--v2" in sys.argv
PFX = "GEMV2" if V2 else "GEMV1"

D = 4            # ring depth: up to D - 1 tiles requested ahead of the one being consumed
VBASE_TOP = 128  # registers are allocated downwards from v127
SBASE = 40       # first SGPR owned by the block


class Regs:
    def __init__(self):
        self.map = {}
        self.next = 0

    def alloc(self, name, n=1, align=1):
        while self.next % align:
            self.next += 1
        self.map[name] = self.next
        self.next += n


def build_regs():
    r = Regs()
    for s in range(D):
        r.alloc("W%d" % s, 4, 4)
    for s in range(2):
        r.alloc("Q%d" % s, 2, 2)  # (qparam word, zero) of the tiles of even / odd ring position
    r.alloc("x", 16, 4)
    for b in "AB":
        r.alloc("c1" + b, 4, 4)
        r.alloc("c2" + b, 4, 4)
        r.alloc("a1" + b, 2, 2)
        r.alloc("a2" + b, 2, 2)
    r.alloc("d", 4, 4)
    r.alloc("uu", 4, 4)
    r.alloc("acc", 4, 4)
    r.alloc("p0", 2, 2)
    r.alloc("p1", 2, 2)
    r.alloc("t", 2, 2)
    r.alloc("wv0", 2, 2)
    r.alloc("wv1", 2, 2)
    r.alloc("m16", 2, 2)  # (fp16 mantissa of the scale, zero)
    r.alloc("ws")
    r.alloc("tt")
    r.alloc("ee")
    r.alloc("xa")
    r.alloc("qx")
    if V2:
        r.alloc("xn")   # LDS address of the next tile's activations
        r.alloc("rd")   # LDS address of the wave's next slot of partial sums
        r.alloc("fl")
    total = r.next
    total += total % 2
    base = VBASE_TOP - total
    base -= base % 4
    for k in r.map:
        r.map[k] += base
    return r.map, base


REG, VBASE = build_regs()
SREG = {n: SBASE + i for i, n in enumerate(
    ["wp_lo", "wp_hi", "ldi", "ntm1", "rem", "c3c00", "cur", "t0"] +
    (["ktn", "kbx", "urem", "ut", "m1_lo", "m1_hi", "m2_lo", "m2_hi", "m3_lo", "m3_hi", "fflag"] if V2 else []))}


# v2: ktn = K tile index of the run's first tile (on entry), kbx = K tiles per row block, urem = tiles of the first
# unit that belong to this run or lie behind it (tiles until the first unit boundary), ut = tiles per unit
SCALAR_INPUTS = ("wp_lo", "wp_hi", "ldi", "ntm1") + (("ktn", "kbx", "urem", "ut") if V2 else ())


def v(name, off=0):
    return "v%d" % (REG[name] + off)


def vv(name, n, off=0):
    return "v[%d:%d]" % (REG[name] + off, REG[name] + off + n - 1)


def s(name):
    return "s%d" % SREG[name]


def ss(name):
    return "s[%d:%d]" % (SREG[name + "_lo"], SREG[name + "_lo"] + 1)


QP_A = "quad_perm:[0,1,0,1] row_mask:0xf bank_mask:0xf"
QP_B = "quad_perm:[2,3,2,3] row_mask:0xf bank_mask:0xf"


def setup_instrs(slot, buf):
    """parameters of the tile in ring slot `slot` into parameter buffer `buf`"""
    q = "Q%d" % (slot % 2)
    return [
        "v_and_b32 %s, 0x7f, %s" % (v("tt"), v(q)),
        "v_lshl_or_b32 %s, %s, 3, %s" % (v("m16"), v("tt"), s("c3c00")),
        "v_perm_b32 %s, %s, %s, %%[sello]" % (v("a1" + buf), v("m16"), v("m16")),
        "v_perm_b32 %s, %s, %s, %%[selhi]" % (v("a1" + buf, 1), v("m16"), v("m16")),
        "v_and_b32 %s, 0xff80, %s" % (v("ee"), v(q)),
        "v_mfma_f32_4x4x4_16b_f16 %s, %s, %%[bc1], 0" % (vv("c1" + buf, 4), vv("m16", 2)),
        "v_perm_b32 %s, %s, %s, %%[sello]" % (v("a2" + buf), v("ee"), v("ee")),
        "v_perm_b32 %s, %s, %s, %%[selhi]" % (v("a2" + buf, 1), v("ee"), v("ee")),
        "v_mfma_f32_4x4x4_16b_bf16 %s, %s, %%[bc2], 0" % (vv("c2" + buf, 4), vv(q, 2)),
    ]


def issue_load(slot):
    """request the next tile of the run into ring slot `slot`, unless the whole run has been requested (a repeated
    request of the last tile would be served by memory again)"""
    return [
        "s_cmp_lt_u32 %s, %s" % (s("ldi"), s("ntm1")),
        "s_cbranch_scc0 20f",
        "s_add_u32 %s, %s, 1" % (s("ldi"), s("ldi")),
        "s_add_u32 %s, %s, 0x400" % (s("wp_lo"), s("wp_lo")),
        "s_addc_u32 %s, %s, 0" % (s("wp_hi"), s("wp_hi")),
        "global_load_dwordx4 %s, %%[woff], %s nt" % (vv("W%d" % slot, 4), ss("wp")),
        "20:",
    ]


def wait_next_tile():
    """wait until the tile after the current one (index cur + 1) has arrived: loads return in order, one load per tile,
    so at most ldi - cur - 1 of them (the tiles requested after it) may still be outstanding.  s_waitcnt takes an
    immediate, hence the ladder; in the steady state the first rung is taken."""
    L = ["s_sub_u32 %s, %s, %s" % (s("t0"), s("ldi"), s("cur"))]   # allowed + 1, 0 .. D - 1 (0 and 1 both mean: wait for all)
    for k in range(D - 1, 1, -1):
        L += ["s_cmp_lt_u32 %s, %d" % (s("t0"), k), "s_cbranch_scc1 %df" % (30 + k), "s_waitcnt vmcnt(%d)" % (k - 1), "s_branch 30f",
              "%d:" % (30 + k)]
    L += ["s_waitcnt vmcnt(0)", "30:"]
    return L


QP_SWAP1 = "quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf"
QP_SWAP2 = "quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf"


def flush(final):
    """v2: the accumulator's row sums -> the wave's next slot of partial sums.  Element l % 4 of the accumulator is the
    lane's own dot product (times f); the sum over the four lanes of a row uses the same operations in the same order
    as the kernel's own reduction, so a run that crosses no boundary gives the same bits either way."""
    L = [
        "v_cndmask_b32 %s, %s, %s, s[%d:%d]" % (v("fl"), v("acc", 0), v("acc", 1), SREG["m1_lo"], SREG["m1_hi"]),
        "v_cndmask_b32 %s, %s, %s, s[%d:%d]" % (v("fl"), v("fl"), v("acc", 2), SREG["m2_lo"], SREG["m2_hi"]),
        "v_cndmask_b32 %s, %s, %s, s[%d:%d]" % (v("fl"), v("fl"), v("acc", 3), SREG["m3_lo"], SREG["m3_hi"]),
        "v_mul_f32 %s, %s, %%[finv]" % (v("fl"), v("fl")),
        "s_nop 1",
        "v_add_f32_dpp %s, %s, %s %s" % (v("fl"), v("fl"), v("fl"), QP_SWAP1),
        "s_nop 1",
        "v_add_f32_dpp %s, %s, %s %s" % (v("fl"), v("fl"), v("fl"), QP_SWAP2),
        "ds_write_b32 %s, %s" % (v("rd"), v("fl")),
    ]
    if not final:
        L.append("v_add_u32 %s, 256, %s" % (v("rd"), v("rd")))
        for i in range(4):
            L.append("v_mov_b32 %s, 0" % v("acc", i))
    return L


def next_x_address():
    """v2, end of a tile: the next tile becomes the current one; K tile index of the one after it, wrapped at the end of
    the row block"""
    return [
        "v_mov_b32 %s, %s" % (v("xa"), v("xn")),
        "s_add_u32 %s, %s, 1" % (s("ktn"), s("ktn")),
        "s_cmp_eq_u32 %s, %s" % (s("ktn"), s("kbx")),
        "s_cselect_b32 %s, 0, %s" % (s("ktn"), s("ktn")),
        "v_lshl_add_u32 %s, %s, 8, %%[xlane]" % (v("xn"), s("ktn")),
    ]


def unit_bookkeeping():
    """v2, after a tile: one tile less in the current unit; at its end arm the flush that the next tile runs"""
    return [
        "s_sub_u32 %s, %s, 1" % (s("urem"), s("urem")),
        "s_cmp_eq_u32 %s, 0" % s("urem"),
        "s_cbranch_scc0 42f",
        "s_mov_b32 %s, 1" % s("fflag"),
        "s_mov_b32 %s, %s" % (s("urem"), s("ut")),
        "42:",
    ]


def tile_body(pos, first):
    """the 8 steps of the tile in ring slot `pos`; `first`: the pipeline is empty (stages of earlier quads are idle)"""
    cur = "AB"[pos % 2]
    prv = "AB"[(pos + 1) % 2]
    nslot = (pos + 1) % D
    L = []
    L += issue_load((pos + D - 1) % D)
    setup = setup_instrs(nslot, prv)
    for u in range(8):
        if u == 3:
            L.append("s_waitcnt lgkmcnt(0)")
            L.append("ds_read_b128 %s, %s offset:%d" % (vv("x", 4, 8), v("xa"), 128 if V2 else pos * 256 + 128))
            L.append("ds_read_b128 %s, %s offset:%d" % (vv("x", 4, 12), v("xa"), 192 if V2 else pos * 256 + 192))
            # (scale, zero) of the tile after the next one (its register's previous content was last read a tile ago)
            L.append("ds_read_b32 %s, %s offset:%d" % (v("Q%d" % (pos % 2)), v("qx"), (pos + 2) * 128))
            if V2 and not first:
                # the previous tile closed a unit: its last product ran in step 2, park its sums before P(0)
                L += ["s_cmp_eq_u32 %s, 0" % s("fflag"), "s_cbranch_scc1 41f"] + flush(False) + ["s_mov_b32 %s, 0" % s("fflag"), "41:"]
        if u == 7:
            L.append("s_waitcnt lgkmcnt(0)")
            L += wait_next_tile()   # X(8) below reads the next tile's first dword
        # M1(u)
        L.append("v_mfma_f32_4x4x4_16b_f16 %s, %s, %s, %s" % (vv("d", 4), vv("a1" + cur, 2), vv("p%d" % (u % 2), 2), vv("c1" + cur, 4)))
        # X(u + 1)
        nu = u + 1
        pn = "p%d" % (nu % 2)
        if nu % 2 == 0:
            wsrc = v("W%d" % nslot, 0) if nu == 8 else v("W%d" % pos, nu // 2)
            L.append("v_lshrrev_b32 %s, 8, %s" % (v("ws"), wsrc))
            src = wsrc
        else:
            src = v("ws")
        L.append("v_and_b32_dpp %s, %s, %%[mask] %s" % (v(pn), src, QP_A))
        L.append("v_and_b32_dpp %s, %s, %%[mask] %s" % (v(pn, 1), src, QP_B))
        # P(u - 3)
        if first and u < 3:
            L.append("s_nop 0")
        else:
            L.append("v_mfma_f32_4x4x4_16b_bf16 %s, %s, %s, %s" % (vv("acc", 4), vv("x", 2, 2 * ((u - 3) % 8)), vv("wv%d" % ((u - 3) % 2), 2), vv("acc", 4)))
        # R2(u - 2)
        if first and u < 2:
            L += ["s_nop 0", "s_nop 0"]
        else:
            wvn = "wv%d" % ((u - 2) % 2)
            L.append("v_cvt_pk_bf16_f32 %s, %s, %s" % (v(wvn), v("uu", 0), v("uu", 1)))
            L.append("v_cvt_pk_bf16_f32 %s, %s, %s" % (v(wvn, 1), v("uu", 2), v("uu", 3)))
        # M2(u - 1)
        if first and u < 1:
            L.append("s_nop 0")
        else:
            sb = cur if u >= 1 else prv
            L.append("v_mfma_f32_4x4x4_16b_bf16 %s, %s, %s, %s" % (vv("uu", 4), vv("a2" + sb, 2), vv("t", 2), vv("c2" + sb, 4)))
        # R1(u)
        L.append("v_cvt_pk_bf16_f32 %s, %s, %s" % (v("t"), v("d", 0), v("d", 1)))
        L.append("v_cvt_pk_bf16_f32 %s, %s, %s" % (v("t", 1), v("d", 2), v("d", 3)))
        # parameters of the next tile
        L.append(setup[u])
        if u == 7:
            L.append(setup[8])
            # first half of the next tile's activations (its registers were last read by P(3) in step 6)
            if V2:
                L.append("ds_read_b128 %s, %s offset:0" % (vv("x", 4, 0), v("xn")))
                L.append("ds_read_b128 %s, %s offset:64" % (vv("x", 4, 4), v("xn")))
                L += next_x_address()
            else:
                L.append("ds_read_b128 %s, %s offset:%d" % (vv("x", 4, 0), v("xa"), (pos + 1) * 256))
                L.append("ds_read_b128 %s, %s offset:%d" % (vv("x", 4, 4), v("xa"), (pos + 1) * 256 + 64))
    return L


def drain(par):
    """the stages still in flight after the last tile (ring position parity `par`)"""
    cur = "AB"[par]
    L = []
    # step 8: P(5), R2(6), M2(7)
    L.append("v_mfma_f32_4x4x4_16b_bf16 %s, %s, %s, %s" % (vv("acc", 4), vv("x", 2, 10), vv("wv1", 2), vv("acc", 4)))
    L.append("v_cvt_pk_bf16_f32 %s, %s, %s" % (v("wv0"), v("uu", 0), v("uu", 1)))
    L.append("v_cvt_pk_bf16_f32 %s, %s, %s" % (v("wv0", 1), v("uu", 2), v("uu", 3)))
    L.append("v_mfma_f32_4x4x4_16b_bf16 %s, %s, %s, %s" % (vv("uu", 4), vv("a2" + cur, 2), vv("t", 2), vv("c2" + cur, 4)))
    # step 9: P(6), R2(7)
    L.append("s_nop 1")
    L.append("v_mfma_f32_4x4x4_16b_bf16 %s, %s, %s, %s" % (vv("acc", 4), vv("x", 2, 12), vv("wv0", 2), vv("acc", 4)))
    L.append("s_nop 3")
    L.append("v_cvt_pk_bf16_f32 %s, %s, %s" % (v("wv1"), v("uu", 0), v("uu", 1)))
    L.append("v_cvt_pk_bf16_f32 %s, %s, %s" % (v("wv1", 1), v("uu", 2), v("uu", 3)))
    # step 10: P(7)
    L.append("s_nop 1")
    L.append("v_mfma_f32_4x4x4_16b_bf16 %s, %s, %s, %s" % (vv("acc", 4), vv("x", 2, 14), vv("wv1", 2), vv("acc", 4)))
    L.append("s_nop 7")
    L.append("s_branch 9f")
    return L


def program():
    L = []
    # ---- preamble.  The caller passes, in the block's own scalar registers: wp = address of the last tile it
    # requested (tile ldi = min(nt - 1, D - 2) of the run), ldi, nt - 1
    L.append("s_mov_b32 %s, 0x3c00" % s("c3c00"))
    L.append("s_add_u32 %s, %s, 1" % (s("rem"), s("ntm1")))
    L.append("s_mov_b32 %s, 0" % s("cur"))
    if V2:
        # lane masks of the lanes 1, 2, 3 of every 4-lane block, the flush flag, the first two activation addresses
        for k, pat in (("m1", 0x22222222), ("m2", 0x44444444), ("m3", 0x88888888)):
            L.append("s_mov_b32 %s, 0x%x" % (s(k + "_lo"), pat))
            L.append("s_mov_b32 %s, 0x%x" % (s(k + "_hi"), pat))
        L.append("s_mov_b32 %s, 0" % s("fflag"))
        L.append("v_mov_b32 %s, %%[redaddr]" % v("rd"))
        L.append("v_lshl_add_u32 %s, %s, 8, %%[xlane]" % (v("xa"), s("ktn")))
        L += ["s_add_u32 %s, %s, 1" % (s("ktn"), s("ktn")), "s_cmp_eq_u32 %s, %s" % (s("ktn"), s("kbx")),
              "s_cselect_b32 %s, 0, %s" % (s("ktn"), s("ktn")),
              "v_lshl_add_u32 %s, %s, 8, %%[xlane]" % (v("xn"), s("ktn"))]
    else:
        L.append("v_mov_b32 %s, %%[xaddr]" % v("xa"))
    L.append("v_mov_b32 %s, %%[qaddr]" % v("qx"))
    L.append("v_mov_b32 %s, 0" % v("m16", 1))
    for sl in range(2):
        L.append("v_mov_b32 %s, 0" % v("Q%d" % sl, 1))
    for i in range(4):
        L.append("v_mov_b32 %s, 0" % v("acc", i))
    L.append("ds_read_b128 %s, %s offset:0" % (vv("x", 4, 0), v("xa")))
    L.append("ds_read_b128 %s, %s offset:64" % (vv("x", 4, 4), v("xa")))
    L.append("ds_read_b32 %s, %s offset:0" % (v("Q0"), v("qx")))
    L.append("ds_read_b32 %s, %s offset:128" % (v("Q1"), v("qx")))
    L.append("s_waitcnt vmcnt(%d) lgkmcnt(0)" % (D - 2))  # tile 0 and the first two qparam words have arrived
    su = setup_instrs(0, "A")
    L += [su[0], su[1], su[2], su[3], su[4], su[6], su[7], "s_nop 1", su[5], su[8]]
    L.append("v_lshrrev_b32 %s, 8, %s" % (v("ws"), v("W0", 0)))
    L.append("v_and_b32_dpp %s, %s, %%[mask] %s" % (v("p0"), v("W0", 0), QP_A))
    L.append("v_and_b32_dpp %s, %s, %%[mask] %s" % (v("p0", 1), v("W0", 0), QP_B))
    L.append("s_nop 7")
    # ---- first tile, then the ring
    L += tile_body(0, True)
    if V2:
        L += unit_bookkeeping()
    L += ["s_add_u32 %s, %s, 1" % (s("cur"), s("cur")), "s_sub_u32 %s, %s, 1" % (s("rem"), s("rem")), "s_cmp_eq_u32 %s, 0" % s("rem"), "s_cbranch_scc1 70f", "s_branch 11f"]
    L.append("10:")
    for pos in range(D):
        if pos == 1:
            L.append("11:")
        L += tile_body(pos, False)
        if V2:
            L += unit_bookkeeping()
        L += ["s_add_u32 %s, %s, 1" % (s("cur"), s("cur")), "s_sub_u32 %s, %s, 1" % (s("rem"), s("rem")), "s_cmp_eq_u32 %s, 0" % s("rem"), "s_cbranch_scc1 %df" % (70 + pos % 2)]
    if not V2:
        L.append("v_add_u32 %s, %d, %s" % (v("xa"), D * 256, v("xa")))
    L.append("v_add_u32 %s, %d, %s" % (v("qx"), D * 128, v("qx")))
    L.append("s_branch 10b")
    L.append("70:")
    L += drain(0)
    L.append("71:")
    L += drain(1)
    L.append("9:")
    if V2:
        L += flush(True)
    L.append("s_waitcnt vmcnt(0) lgkmcnt(0)")  # repeated requests of the last tile and the next tile's activations
    return L


def clobbers():
    regs = []
    ring = set()
    for sl in range(D - 1):
        ring |= set(range(REG["W%d" % sl], REG["W%d" % sl] + 4))
    acc = set() if V2 else set(range(REG["acc"], REG["acc"] + 4))
    for i in range(VBASE, VBASE_TOP):
        if i not in ring and i not in acc:
            regs.append('"v%d"' % i)
    for name, n in SREG.items():
        if name not in SCALAR_INPUTS:
            regs.append('"s%d"' % n)
    regs += ['"scc"', '"memory"']
    return regs


def main():
    out = []
    out.append("// Generated by gen_int4wo_gemv1.py -- do not edit; see that script for the schedule.")
    out.append("#ifndef %s_RING_DEPTH" % PFX)
    out.append("#define %s_RING_DEPTH %d" % (PFX, D))
    out.append("#define %s_VBASE %d" % (PFX, VBASE))
    out.append("#define %s_S_WP \"{s[%d:%d]}\"" % (PFX, SREG["wp_lo"], SREG["wp_hi"]))
    for n in SCALAR_INPUTS[2:]:
        out.append("#define %s_S_%s \"{s%d}\"" % (PFX, n.upper(), SREG[n]))
    for sl in range(D):
        out.append("#define %s_W%d \"{v[%d:%d]}\"" % (PFX, sl, REG["W%d" % sl], REG["W%d" % sl] + 3))
    out.append("#define %s_ACC \"{v[%d:%d]}\"" % (PFX, REG["acc"], REG["acc"] + 3))
    out.append("#define %s_CLOBBERS " % PFX + ", ".join(clobbers()))
    out.append("#define %s_LOOP_ASM \\" % PFX)
    for l in program():
        out.append('    "%s\\n\\t" \\' % l)
    out.append('    ""')
    out.append("#endif")
    print("\n".join(out))


if __name__ == "__main__":
    main()
