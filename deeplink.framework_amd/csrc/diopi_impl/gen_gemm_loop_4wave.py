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

One tile of the loop (stage s = tile & 1), 128 MFMAs:
  k-step 0: 64 MFMAs out of fragment buffer 0 | the 16 fragment reads of k-step 1 (stage s) into buffer 1
  s_waitcnt vmcnt(0) lgkmcnt(0); s_barrier    every wave is done reading stage s, tile t + 1 has landed in stage s ^ 1
  k-step 1: 64 MFMAs out of buffer 1 | the 16 fragment reads of tile t + 1, k-step 0 into buffer 0
                                     | the 16 loads of tile t + 2 into stage s, spread over the whole k-step
Fragment reads are issued in the order the MFMAs need them (B0, A0..A7, B1..B7; the MFMAs run B-major) and LDS
returns them in order, so the wait before an MFMA is a count of younger reads that may still be outstanding.
Measured on 8192 x 4096 x 11008: issuing the loads later (half of them in the next k-step 0) or packed into the
first half of k-step 1 is 5-10 % slower; every third MFMA slot for the reads against every second: no difference."""
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


def kstep(out, buf, prefetch, load_stage):
    """64 MFMAs out of fragment buffer `buf`; prefetch = (stage, ks) read into the other buffer or None;
    load_stage = stage that receives the 16 loads of the tile at %[kcur], or None."""
    after = {m: [] for m in range(64)}
    reads_before = [0] * 64
    if prefetch:
        slots = [1 + 3 * r for r in range(16)]
        for r, slot in enumerate(slots):
            after[slot].append(("read", r))
        reads_before = [sum(1 for slot in slots if slot < m) for m in range(64)]
    if load_stage is not None:
        for d in range(16):
            slot = 2 + (d * 60) // 16
            after[slot].append(("m0", d))          # M0 is written one MFMA before the load that reads it
            after[slot + 1].append(("load", d))
    waited = -1
    for j in range(8):
        for i in range(8):
            m = j * 8 + i
            need = READ_ORDER.index(("A", 7)) if j == 0 else READ_ORDER.index(("B", j))
            if need > waited:
                out.append(f"s_waitcnt lgkmcnt({min(15 - need + reads_before[m], 15)})")
                waited = need
            out.append(f"MFMA {acc(i, j)}, {vb(buf, j)}, {va(buf, i)}, {acc(i, j)}")
            for what, arg in after[m]:
                if what == "read":
                    read_fragment(out, READ_ORDER[arg][0], READ_ORDER[arg][1], 1 - buf, prefetch[0], prefetch[1])
                elif what == "m0":
                    load_m0(out, arg, load_stage)
                else:
                    load_issue(out, arg)


def tile(out, s, loads, next_tile):
    kstep(out, 0, (s, 1), None)
    out.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
    out.append("s_barrier")
    kstep(out, 1, (s ^ 1, 0) if next_tile else None, s if loads else None)


def prologue(out):
    out.append("s_mov_b32 %[m0s], m0")
    for stage in (0, 1):                            # tiles 0 and 1
        for d in range(16):
            load_m0(out, d, stage)
            out.append("s_nop 0")
            load_issue(out, d)
    for r in range(256):                            # while the loads are in flight
        out.append(f"v_accvgpr_write_b32 a{r}, 0")
    out.append("s_waitcnt vmcnt(16)")               # tile 0 has landed
    out.append("s_barrier")
    for kind, idx in READ_ORDER:
        read_fragment(out, kind, idx, 0, 0, 0)


def main():
    pro, body, tail = [], [], []
    prologue(pro)
    tile(body, 0, True, True)
    tile(body, 1, True, True)
    tile(tail, 0, False, True)
    tile(tail, 1, False, False)
    tail += ["s_nop 15", "s_nop 15", "s_mov_b32 m0, %[m0s]"]   # the last MFMAs have written their accumulators
    clobbers = ", ".join(f'"v{r}"' for r in range(VA0, VA0 + 128)) + ", " + ", ".join(f'"a{r}"' for r in range(256))
    text = ["// Generated by gen_gemm_loop_4wave.py (see there for the schedule); do not edit.\n"]
    for name, lines in (("PROLOGUE", pro), ("BODY", body), ("TAIL", tail)):
        for suffix, mnemonic in (("BF16", "v_mfma_f32_16x16x32_bf16"), ("F16", "v_mfma_f32_16x16x32_f16")):
            text.append(f"#define GEMM4W_{name}_{suffix} \\\n")
            text.append(" \\\n".join('  "' + l.replace("MFMA", mnemonic) + '\\n\\t"' for l in lines) + "\n\n")
    text.append(f"#define GEMM4W_CLOBBERS {clobbers}\n")
    path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_loop_4wave.inc")
    with open(path, "w") as f:
        f.write("".join(text))


if __name__ == "__main__":
    main()
