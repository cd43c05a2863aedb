#!/usr/bin/env python3
"""Generates csrc/walk_asm.inc: the inner loop of the conv kernel as inline-assembly strings.

Run `python3 gen_walk_asm.py > walk_asm.inc` after changing it; the output is committed so that the build
needs only hipcc.

One *entry* of a wave's stream is two dwords {code, weight}:
    code[15:0]   byte offset into the lane's LDS region
    code[23:16]  accumulator index (first VGPR of the output channel's 4*NQ accumulators, relative to v128)
    code[31:28]  0xC, so that `code >> 16` written to M0 is at once the VGPR index (M0[7:0]) and the
                 "index the destination and the addend" enables (M0[15:12]) of VGPR index mode
Eight entries (64 bytes) are one scalar fetch.

Register plan (the kernel confines the compiler below A0):
    v[ACC0 .. ACC0+NACC-1]   accumulators (v128..v255, or v64..v127 in the 64-accumulator variant)
    v[X0 + 4*NQ*b ...]       landing buffer b of the LDS reads (NBUF buffers, reads run NBUF-1 entries ahead)
    v[A0 .. A0+7]            LDS addresses of the eight entries of the batch being read
    s36..s51 / s52..s67      current / next batch, s70 = 0xC000 (index 0 + enables), s72:s73 stream address

Variants (macro suffix): ""  one 64 KiB LDS tile, 128 accumulators, 16-bit LDS addresses;
                         "3" three LDS buffers (addresses up to 160 KiB), 128 accumulators;
                         "4" three LDS buffers, 64 accumulators and at most 64 VGPRs below them, so that four
                             waves fit a SIMD (measured: 56 TFLOP/s for the loop alone against 43-50 with two);
                         "5" as "4" with buffers of half the size, for two 8-wave workgroups per CU;
                         "6", "7", "8" as "4", "3", "5" for the flat kernels' LDS buffers of 64 / 64 / 32 KiB.

Per entry the loop issues: NQ ds_read_b128, one s_lshr (M0), one s_waitcnt, 4*NQ v_fma; per batch: one
s_load_dwordx16, eight v_add_u16 (addresses), a handful of scalar ops.
"""

TILE_BYTES = 65536   # LDS tile of the single-buffered kernel
BUF_BYTES = 54272    # one of the three LDS buffers of the triple-buffered kernels (3 * 53 KiB <= 160 KiB)
HALF_BUF_BYTES = 27136  # ... when two workgroups share a CU
FLAT_BUF_BYTES = 65536       # one of the two LDS buffers of the flat (pointwise) kernels
FLAT_HALF_BUF_BYTES = 32768  # ... when two workgroups share a CU

# record sizes to emit loops for: single entries, and pairs of entries that share one set of LDS reads (the same input
# position for two output channels of the wave).  The flat kernels' waves hold few channels: singles only.
SHARES = {"": (1, 2), "3": (1, 2), "4": (1, 2), "5": (1, 2), "6": (1,), "7": (1,), "8": (1,)}

VARIANTS = {
    "": dict(wide=False, acc0=128, nacc=128, nbuf={1: 4, 2: 4, 4: 2}),
    "3": dict(wide=True, acc0=128, nacc=128, nbuf={1: 4, 2: 4, 4: 2}),
    "4": dict(wide=True, acc0=64, nacc=64, nbuf={1: 4, 2: 2}),
    "5": dict(wide=True, acc0=64, nacc=64, nbuf={1: 4, 2: 2}, buf=HALF_BUF_BYTES),
    # flat tiles of pointwise layers: two LDS buffers of 64 KiB (one workgroup per CU) or 32 KiB (two per CU)
    "6": dict(wide=True, acc0=64, nacc=64, nbuf={1: 4, 2: 2}, buf=FLAT_BUF_BYTES),
    "7": dict(wide=True, acc0=128, nacc=128, nbuf={1: 4, 2: 4, 4: 2}, buf=FLAT_BUF_BYTES),
    "8": dict(wide=True, acc0=64, nacc=64, nbuf={1: 4, 2: 2}, buf=FLAT_HALF_BUF_BYTES),
}


def cfg(nq, variant=""):
    """wide: LDS addresses may exceed 64 KiB (triple-buffered kernels), so they are formed in 32 bits."""
    v = VARIANTS[variant]
    nbuf = v["nbuf"][nq]
    x_regs = 4 * nq * nbuf
    a0 = v["acc0"] - x_regs - 8
    return dict(nq=nq, nbuf=nbuf, a0=a0, x0=a0 + 8, ahead=nbuf - 1, wide=v["wide"], acc0=v["acc0"], nacc=v["nacc"],
                region=(v.get("buf", BUF_BYTES) if v["wide"] else TILE_BYTES) // nq)


def reads(c, buf, addr_reg):
    out = []
    for q in range(c["nq"]):
        r = c["x0"] + 4 * c["nq"] * buf + 4 * q
        off = "" if q == 0 else " offset:%d" % (q * c["region"])
        out.append("ds_read_b128 v[%d:%d], v%d%s" % (r, r + 3, addr_reg, off))
    return out


def fmas(c, buf, wreg):
    out = []
    for i in range(4 * c["nq"]):
        out.append("v_fma_f32 v%d, s%d, v%d, v%d" % (c["acc0"] + i, wreg, c["x0"] + 4 * c["nq"] * buf + i, c["acc0"] + i))
    return out


def addresses(c, first_code_reg):
    # under index 0: v[A0+r] = code[15:0] of record r's first entry + lane base (a 16-bit add, or u16 * 1 + u32
    # when the base can exceed 16 bits)
    out = ["s_mov_b32 m0, s70"]
    for r in range(8 // c["share"]):
        src = first_code_reg + 2 * r * c["share"]
        if c["wide"]:
            out.append("v_mad_u32_u16 v%d, s%d, 1, %%[base]" % (c["a0"] + r, src))
        else:
            out.append("v_add_u16 v%d, s%d, %%[base]" % (c["a0"] + r, src))
    return out


def walk(nq, variant="", share=1):
    """share: consecutive entries of the stream come in records of `share` entries that have the same LDS offset
    (the same input position, different output channels), so one set of LDS reads serves `share` entries."""
    c = cfg(nq, variant)
    c["share"] = share
    R = 8 // share                       # records per batch
    nbuf = min(c["nbuf"], R)
    ahead = nbuf - 1                     # records of look-ahead
    L = []
    # the batch (s36..s51) and the stream address (s72:s73) are the asm statement's in/out operands, bound to these very
    # registers by their constraints: no copies in or out
    L.append("s_mov_b32 s70, 0xc000")
    for r in range(R):
        L.append("v_mov_b32 v%d, 0" % (c["a0"] + r))
    L.append("s_set_gpr_idx_on s70, 0xc")
    L += addresses(c, 36)
    for r in range(ahead):  # prime the pipeline
        L += reads(c, r % nbuf, c["a0"] + r)
    # The loop body handles one batch and is unrolled four times; copy k runs at wave priority k.  A wave enters at
    # copy %[ph] (its index on the SIMD plus a running count), so the waves of a SIMD hold different priorities
    # that rotate with every batch.  Left alone the SIMD serves its oldest wave first: that wave finishes its stage
    # early and idles at the barrier while the youngest runs the tail of the stage alone, too slowly to fill the
    # SIMD by itself.
    # A stream is padded to whole batches with entries of weight zero.  With single-entry records the last batch of a
    # call gets a copy of the body of its own (label 5) that leaves at the first zero weight (label 8): pads cost no
    # FMAs.  (Real entries never carry +0.0: only non-zeros are packed.  In a stream of pairs a zero weight also marks
    # the missing half of a pair, so those loops run every entry.)
    last_exits = share == 1
    if last_exits:
        L.append("s_cmp_eq_u32 %[nb], 1")
        L.append("s_cbranch_scc1 5f")
    for k in (1, 2, 3):
        L.append("s_cmp_eq_u32 %%[ph], %d" % k)
        L.append("s_cbranch_scc1 %df" % (k + 1))

    def body(prio, exits):
        L.append("s_setprio %d" % prio)
        L.append("s_load_dwordx16 s[52:67], s[72:73], 0x0")  # the batch after this one (may belong to the next stream)
        L.append("s_add_u32 s72, s72, 64")
        L.append("s_addc_u32 s73, s73, 0")
        refill_at = R - ahead  # first record whose look-ahead record lies in the next batch
        for r in range(R):
            if exits and r > 0:  # (a call is never made for an empty stream: the first entry of a batch is real)
                L.append("s_cmp_eq_u32 s%d, 0" % (37 + 2 * r))
                L.append("s_cbranch_scc1 8f")
            if r == refill_at and not exits:
                # the next batch must have arrived; its addresses replace the ones all consumed by now
                L.append("s_waitcnt lgkmcnt(0)")
                L.extend(addresses(c, 52))
            la = r + ahead  # record whose reads are issued now
            # The last batch of a call reads nothing beyond itself (the next call forms its own addresses and primes
            # its own reads), so its waits count only the reads of its later records; the scalar fetch of the next
            # batch may still be in flight, which only makes such a wait stricter.
            if not exits or la < R:
                L.extend(reads(c, la % nbuf, c["a0"] + (la % R)))
            in_flight = ahead if not exits else min(R - 1, la) - r
            for kk in range(share):
                e = r * share + kk
                L.append("s_lshr_b32 m0, s%d, 16" % (36 + 2 * e))
                if kk == 0:
                    L.append("s_waitcnt lgkmcnt(%d)" % (in_flight * nq))
                else:
                    L.append("s_nop 0")  # keeps one instruction between the write of M0 and the indexed VALU use
                L.extend(fmas(c, r % nbuf, 37 + 2 * e))

    def advance():
        for i in range(8):
            L.append("s_mov_b64 s[%d:%d], s[%d:%d]" % (36 + 2 * i, 37 + 2 * i, 52 + 2 * i, 53 + 2 * i))

    for k in range(4):
        L.append("%d:" % (k + 1))
        body(k, False)
        advance()
        L.append("s_sub_u32 %[nb], %[nb], 1")
        if last_exits:
            L.append("s_cmp_eq_u32 %[nb], 1")
            L.append("s_cbranch_scc1 5f")
            if k == 3:
                L.append("s_branch 1b")
        else:
            L.append("s_cmp_lg_u32 %[nb], 0")
            if k < 3:
                L.append("s_cbranch_scc0 9f")
            else:
                L.append("s_cbranch_scc1 1b")
    if last_exits:
        L.append("5:")
        body(1, True)
        L.append("8:")
        L.append("s_waitcnt lgkmcnt(0)")  # the next batch has arrived (an early exit may come before the refill's wait)
        advance()
    L.append("9:")
    L.append("s_setprio 3")  # what follows a walk (issuing the staging loads, reaching the barrier) should not wait
    L.append("s_waitcnt lgkmcnt(0)")  # drain the look-ahead reads (their data is not used)
    L.append("s_set_gpr_idx_off")
    return c, L


def regs(lo, hi):
    return ", ".join('"v%d"' % r for r in range(lo, hi))


def main():
    print("// Generated by gen_walk_asm.py -- do not edit.")
    for variant, v in VARIANTS.items():
        for nq in sorted(v["nbuf"]):
            for share in SHARES[variant]:
                c, L = walk(nq, variant, share)
                print("#define TETRIS_WALK%s_ASM_%d_S%d \\" % (variant, nq, share))
                for line in L:
                    print('  "%s\\n" \\' % line)
                print('  ""')
            print("#define TETRIS_WALK%s_FIRST_RESERVED_%d %d" % (variant, nq, c["a0"]))
            print("#define TETRIS_WALK%s_VGPR_CLOBBERS_%d %s" % (variant, nq, regs(c["a0"], c["acc0"])))
        print("#define TETRIS_WALK%s_ACC_CLOBBERS %s" % (variant, regs(v["acc0"], v["acc0"] + v["nacc"])))
    print("#define TETRIS_WALK_TILE_BYTES %d" % TILE_BYTES)
    print("#define TETRIS_WALK_BUF_BYTES %d" % BUF_BYTES)
    print("#define TETRIS_WALK_HALF_BUF_BYTES %d" % HALF_BUF_BYTES)
    print("#define TETRIS_WALK_FLAT_BUF_BYTES %d" % FLAT_BUF_BYTES)
    print("#define TETRIS_WALK_FLAT_HALF_BUF_BYTES %d" % FLAT_HALF_BUF_BYTES)


if __name__ == "__main__":
    main()
