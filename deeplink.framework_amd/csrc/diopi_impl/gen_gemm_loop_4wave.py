#!/usr/bin/env python3
"""Writes gemm_loop_4wave.inc: the K loop of the 4-wave 256 x 256 x 64 GEMM kernel (gemm.hip,
gemmMfma4WaveKernel) as inline-assembly text for gfx950.

Why a generator: with one wave per SIMD nothing hides a stall, so every instruction of the loop is placed by hand:
which MFMA an LDS fragment read or a tile load follows, and the exact s_waitcnt before the first MFMA that needs a
fragment. The compiler cannot be told to keep 256 accumulators in fixed accumulation registers across iterations
and to leave the order alone, so the loop is emitted as text with physical register names.

Registers (per lane):   a[0:255]    accumulators, tile (i, j) of the wave's 8 x 8 grid of 16 x 16 at a[4 (8 i + j) ..]
                        v[120:183]  A fragments, two buffers of 8 (one per 32-wide k-step)
                        v[184:247]  B fragments, two buffers of 8
Operands of each block: %[voA0..7] %[voB0..7]  lane byte offsets of the 8 + 8 tile loads of this wave
                        %[adA0] %[adA1] %[adB0] %[adB1]  LDS byte addresses of this lane's fragment chunk for k-step 0 / 1
                        %[rsA] %[rsB]  buffer descriptors, %[lds] LDS address of this wave's 1 KiB slot in stage 0 of A
                        %[kcur]  K byte offset of the tile whose loads are issued next, %[m0s]  the caller's M0

One tile of the loop (stage s = tile & 1), 128 MFMAs, two barriers:
  k-step 0, MFMAs 0-22    out of fragment buffer 0 | the 16 fragment reads of k-step 1 (stage s) into buffer 1, one per MFMA
  s_waitcnt lgkmcnt(0); s_barrier (B1)    every wave is done reading stage s: it may be refilled
  k-step 0, MFMAs 23-63   | the loads of tile t + 2 into stage s start here, one per five MFMAs, and run on into k-step 1
  s_waitcnt vmcnt(loads of tile t + 2 issued so far); s_barrier (B2)    tile t + 1 has landed in stage s ^ 1
  k-step 1, 64 MFMAs out of buffer 1 | the 16 fragment reads of tile t + 1, k-step 0 into buffer 0 | the rest of the loads
A load is needed at B2 of the next tile, so the youngest has more than a whole tile (128 MFMAs, about 1.3 us) to
arrive, at half the issue rate of a schedule that packs the loads between one barrier per tile and the next k-step
boundary: 16.9 cycles per MFMA against 18.2 on 8192 x 4096 x 11008 (16.3 with no tile loads at all). The kernel runs at
the power limit, where the cycles saved come back as a lower clock (1.59 against 1.65 GHz, the same time per launch); they
count when the clock is not what limits it.
Fragment reads are issued in the order the MFMAs need them (B0, A0..A7, B1..B7; the MFMAs run B-major) and LDS
returns them in order, so the wait before an MFMA is a count of younger reads that may still be outstanding.
Within a k-step the A fragments are walked forth for even B fragments and back for odd ones, so consecutive MFMAs
always share one operand (with A0..A7 restarted for every B, both operands change at each turn). At the power limit
that is measurable: 8192 x 4096 x 12288 550.4 -> 545.9 us, x 22016 985.9 -> 978.2 us, same box, same results bit for bit.
Measured and not used: K tiles of 32 in a four-stage ring (loads three tiles ahead) is 10 % slower, because a tile
load then fetches 64-byte row pieces, twice the cache lines per byte; issuing the loads twice as densely (to gain
slack) stalls the wave at issue. The same tile out of v_mfma_f32_32x32x16 (4 x 4 blocks per wave, four 16-wide k-steps,
the same number of fragment reads) takes 1.5 % fewer cycles and 9 % more time (592 -> 646 us on 8192 x 4096 x 12288): that
instruction reads and writes twice the accumulator registers per multiply-add, and at the power limit this is paid in
clock. Register-only loops of either instruction over the whole chip (no memory traffic at all) sustain 2160 TFLOP/s at
2.12 GHz (16x16x32, 16.4 cycles per instruction) against 1940 TFLOP/s at 1.87 GHz (32x32x16, 32.4 cycles): the first
figure is the ceiling that the power limit leaves to any bf16 GEMM here, 0.86 of the nominal peak."""
import os
import sys

READ_ORDER = [("B", 0)] + [("A", i) for i in range(8)] + [("B", j) for j in range(1, 8)]
VA0, VB0 = 120, 184


def va(b, i):
    r = VA0 + b * 32 + i * 4
    return f"v[{r}:{r + 3}]"


def vb(b, j):
    r = VB0 + b * 32 + j * 4
    return f"v[{r}:{r + 3}]"


def acc(i, j):
    r = 4 * (8 * i + j)
    return f"a[{r}:{r + 3}]"


def load_m0(out, d, stage):
    out.append(f"s_add_u32 m0, %[lds], {stage * 32768 + (65536 if d >= 8 else 0) + (d % 8) * 4096}")


def load_issue(out, d):
    is_b = d >= 8
    out.append(f"buffer_load_dwordx4 %[vo{'B' if is_b else 'A'}{d % 8}], %[{'rsB' if is_b else 'rsA'}], %[kcur] offen lds")
    if d == 15:
        out.append("s_add_u32 %[kcur], %[kcur], 128")


def read_fragment(out, kind, idx, buf, stage, ks):
    reg = va(buf, idx) if kind == "A" else vb(buf, idx)
    out.append(f"ds_read_b128 {reg}, %[ad{kind}{ks}] offset:{idx * 2048 + stage * 32768}")


B1_SLOT = 22       # B1 follows this MFMA of k-step 0
LOAD_STEP = 5      # MFMAs between two tile loads


def tile(out, s, loads, next_tile, next_output=False):
    """128 MFMAs of one K tile in stage s; loads: issue the 16 loads of tile t + 2; next_tile: read tile t + 1's first
    fragments during k-step 1; next_output (last K tile of an output tile only): once B1 has freed both stages, issue
    the 32 loads of the first two K tiles of the workgroup's next output tile (the caller passes that tile's lane
    offsets), so that they land while the epilogue runs."""
    after = {m: [] for m in range(128)}
    for r in range(16):                                    # this tile's k-step 1 fragments, right away
        after[r].append(("read1", r))
    after[B1_SLOT].append(("B1", None))
    loads_before_b2 = 0
    if loads:
        for d in range(16):
            slot = B1_SLOT + 1 + d * LOAD_STEP
            if slot + 1 <= 63:
                loads_before_b2 += 1
            after[slot].append(("m0", d))                  # M0 is written one MFMA before the load that reads it
            after[slot + 1].append(("load", d))
    if next_output:
        after[B1_SLOT].append(("rewind", None))
        for n in range(32):
            slot = B1_SLOT + 1 + n * 3
            after[slot].append(("m0n", n))
            after[slot + 1].append(("load", n % 16))
    if next_tile:
        for r in range(16):
            after[65 + 3 * r].append(("read0", r))
    for m in range(128):
        ks, mm = divmod(m, 64)
        j, pos = divmod(mm, 8)
        i = pos if j % 2 == 0 else 7 - pos                 # A fragments back and forth: one operand changes per MFMA
        if m == 0:
            out.append("s_waitcnt lgkmcnt(7)")             # B0, A0..A7 of buffer 0 (read during the previous k-step 1)
        elif ks == 0 and pos == 0 and j >= 1 and m <= B1_SLOT:
            # B_j of buffer 0: 7 - j reads of its set are younger, and so are this tile's reads issued so far
            out.append(f"s_waitcnt lgkmcnt({min(7 - j + min(m, 16), 15)})")
        if m == 64 and next_tile:                          # B2; the last K tile has no successor to wait for
            out.append(f"s_waitcnt vmcnt({loads_before_b2}) lgkmcnt(0)")
            out.append("s_barrier")
        out.append(f"MFMA {acc(i, j)}, {vb(ks, j)}, {va(ks, i)}, {acc(i, j)}")
        for what, arg in after[m]:
            if what == "read1":
                read_fragment(out, READ_ORDER[arg][0], READ_ORDER[arg][1], 1, s, 1)
            elif what == "read0":
                read_fragment(out, READ_ORDER[arg][0], READ_ORDER[arg][1], 0, s ^ 1, 0)
            elif what == "B1":
                out.append("s_waitcnt lgkmcnt(0)")
                out.append("s_barrier")
            elif what == "m0":
                load_m0(out, arg, s)
            elif what == "m0n":
                load_m0(out, arg % 16, arg // 16)
            elif what == "rewind":
                out.append("s_mov_b32 %[kcur], 0")
            else:
                load_issue(out, arg)


def prologue(out, issue_loads):
    """issue_loads: issue the loads of K tiles 0 and 1 (otherwise the workgroup's previous output tile did, before its
    epilogue). The wait that follows allows 16 operations to be outstanding. Loads return in order, so whatever else
    is still counted (K tile 1's 16 loads, the previous epilogue's stores), K tile 0 has landed: if one of its
    loads were pending, all 16 younger loads of K tile 1 would be too."""
    out.append("s_mov_b32 %[m0s], m0")
    if issue_loads:
        for stage in (0, 1):
            for d in range(16):
                load_m0(out, d, stage)
                out.append("s_nop 0")
                load_issue(out, d)
    for r in range(256):                            # while the loads are in flight
        out.append(f"v_accvgpr_write_b32 a{r}, 0")
    out.append("s_waitcnt vmcnt(16)")
    out.append("s_barrier")
    for kind, idx in READ_ORDER:
        read_fragment(out, kind, idx, 0, 0, 0)


def main():
    pro, proc, body, tail, tailn = [], [], [], [], []
    prologue(pro, True)
    prologue(proc, False)
    tile(body, 0, True, True)
    tile(body, 1, True, True)
    for t, nxt in ((tail, False), (tailn, True)):
        tile(t, 0, False, True)
        tile(t, 1, False, False, nxt)
        t += ["s_nop 15", "s_nop 15", "s_mov_b32 m0, %[m0s]"]   # the last MFMAs have written their accumulators
    clobbers = ", ".join(f'"v{r}"' for r in range(VA0, VA0 + 128)) + ", " + ", ".join(f'"a{r}"' for r in range(256))
    text = ["// Generated by gen_gemm_loop_4wave.py (see there for the schedule); do not edit.\n"]
    for name, lines in (("PROLOGUE", pro), ("PROLOGUE_LOADED", proc), ("BODY", body), ("TAIL", tail), ("TAIL_NEXT", tailn)):
        for suffix, mnemonic in (("BF16", "v_mfma_f32_16x16x32_bf16"), ("F16", "v_mfma_f32_16x16x32_f16")):
            text.append(f"#define GEMM4W_{name}_{suffix} \\\n")
            text.append(" \\\n".join('  "' + l.replace("MFMA", mnemonic) + '\\n\\t"' for l in lines) + "\n\n")
    text.append(f"#define GEMM4W_CLOBBERS {clobbers}\n")
    path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_loop_4wave.inc")
    with open(path, "w") as f:
        f.write("".join(text))


if __name__ == "__main__":
    main()
