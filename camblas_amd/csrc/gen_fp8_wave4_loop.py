#!/usr/bin/env python3
"""Writes fp8_wave4_loop_192x256.inc: the K loop of fp8_wave4.hip as inline-assembly statements.

The FP8 block-scaled prefill linear (1x128 activation groups, 128x128 weight blocks, FP32 scales;
rule: per 128-wide K group the unscaled dot product on the matrix cores, then
acc = fma(dot, a_s * w_s, acc) with the product of the scales rounded first, groups ascending) on
four wavefronts per workgroup, one per SIMD. A workgroup owns 192 weight rows x 256 tokens, a
wavefront 96 x 128: 6 x 8 tiles of v_mfma_scale_f32_16x16x128_f8f6f4 (unit hardware scales), one
instruction per tile and K group.

Register plan of a wavefront (nothing is left to the allocator inside the loop):
  v0..v191    the 48 accumulator tiles (the scaled accumulate is vector-ALU work, which cannot touch
              the accumulation registers, so the accumulators live in the architectural half)
  v192..v207  four temporaries for unscaled dot products (ring: the tile's dot is scaled two tiles later)
  v208..v223  a_s * w_s of the current group for the wavefront's eight token tiles, two sets: the 96
              weight rows of a wavefront lie in at most two 128-row scale blocks, tiles below SPLIT
              use set 0, the others set 1 (three variants of the loop: SPLIT 2, 4 and 6 = one block)
  v224..v233  the next group's activation scales (8) and weight scales (2), read from LDS slabs
  a0..a223    the operand fragments, double-buffered per K group (LDS reads land in accumulation
              registers directly, and the matrix instruction takes its A and B operands from them)
One K group (step) of a wavefront: 48 matrix instructions back to back; behind each the four scaled
accumulates of the tile two before it, and spread between them the LDS reads of the next group's
fragments into the other fragment buffer, its scales, and the 14 direct-to-LDS fills of the group
after that into the LDS stage that group's fragments were read from a step ago. Then one wait and
one barrier. Every eighth group the next eight groups' scales are copied into LDS slabs (16 bytes
per lane, direct to LDS), so that a lane finds its eight tokens' scales with eight 4-byte LDS reads.

The fragment file uses local variables of the including function by name (see fp8_wave4.hip).
Usage: python gen_fp8_wave4_loop.py [--out DIR]
"""

import argparse
from pathlib import Path

NA, NB = 6, 8  # 16-row weight tiles and 16-token tiles per wavefront
TILES = NA * NB
STAGE = (32 * NA + 256) * 128  # bytes of one LDS stage: 192 weight rows then 256 token rows of 128 bytes
A_SLAB = 2 * STAGE  # two buffers of [256 tokens][8 groups] floats, 8 KB each, 8 KB apart
W_SLAB = A_SLAB + 16384  # two buffers of [8 blocks][8 groups] floats, 256 bytes each
FILLS = NA + NB  # direct-to-LDS loads per wavefront and step
FRAG = 8 * (NA + NB)  # accumulation registers of one fragment buffer

DOT, PROD, NEXT_A, NEXT_W, UNIT, STAGE1, SCRATCH = 192, 208, 224, 232, 234, 235, 239
SAVED_M0, OFFSET, FILL1, SLAB_TARGET, W_TARGET = "s84", "s85", "s86", "s87", "s88"


def acc(i, j):
    base = 4 * (i * NB + j)
    return f"v[{base}:{base + 3}]"


def a_frag(buffer, i):
    return buffer * FRAG + 8 * i


def b_frag(buffer, j):
    return buffer * FRAG + 8 * (NA + j)


def fragment_reads(stage, buffer):
    """LDS reads of one group's fragments into accumulation registers: per 16-row tile the 16 bytes at
    chunk c and at chunk 4 + c of the lane's row (c = lane / 16), which the XOR swizzle turns into two
    lane addresses per operand."""
    if stage == 0:
        names = ("%[ra_lo]", "%[ra_hi]", "%[rb_lo]", "%[rb_hi]")
    else:
        names = tuple(f"v{STAGE1 + n}" for n in range(4))
    lines = []
    for i in range(NA):
        r = a_frag(buffer, i)
        lines.append(f"ds_read_b128 a[{r}:{r + 3}], {names[0]} offset:{i * 2048}")
        lines.append(f"ds_read_b128 a[{r + 4}:{r + 7}], {names[1]} offset:{i * 2048}")
    for j in range(NB):
        r = b_frag(buffer, j)
        lines.append(f"ds_read_b128 a[{r}:{r + 3}], {names[2]} offset:{j * 2048}")
        lines.append(f"ds_read_b128 a[{r + 4}:{r + 7}], {names[3]} offset:{j * 2048}")
    return lines


def scale_reads():
    """The next group's scales from the slabs: the lane's eight tokens (16 apart: 512 bytes apart in a
    slab of [token][8 groups]) and the wavefront's two weight blocks."""
    lines = [f"ds_read_b32 v{NEXT_A + j}, %[sa] offset:{512 * j}" for j in range(NB)]
    lines += [f"ds_read_b32 v{NEXT_W}, %[sw]", f"ds_read_b32 v{NEXT_W + 1}, %[sw] offset:32"]
    return lines


def fill_units(target):
    """Per direct-to-LDS load: (scalar set-up, the load). M0 walks the wavefront's LDS slots in 4 KB
    strides through the weight rows and on into the token rows; the row advance of successive loads is
    the scalar offset (both operands have rows of K bytes)."""
    units = []
    for n in range(FILLS):
        weights = n < NA
        first = n == 0 or n == NA
        second = n == 1 or n == NA + 1
        lane, resource = ("%[a_off]", "%[rsrc_a]") if weights else ("%[b_off]", "%[rsrc_b]")
        before = [f"s_mov_b32 m0, {target}" if n == 0 else "s_add_u32 m0, m0, 0x1000"]
        if second:
            before.append(f"s_mov_b32 {OFFSET}, %[row_step]")
        elif not first:
            before.append(f"s_add_u32 {OFFSET}, {OFFSET}, %[row_step]")
        units.append((before, f"buffer_load_dwordx4 {lane}, {resource}, {'0' if first else OFFSET} offen lds"))
    return units


ADVANCE = ["v_add_u32_e32 %[a_off], 0x80, %[a_off]", "v_add_u32_e32 %[b_off], 0x80, %[b_off]"]


def slab_loads():
    """The next eight groups' scales into the slab buffers that are not being read: two pieces of the
    activation slab per wavefront (32 tokens each, lanes 2t and 2t + 1 bring groups 0-3 and 4-7 of token
    t) and the weight-block slab (every wavefront brings the same bytes to the same place)."""
    return [
        f"s_mov_b32 m0, {SLAB_TARGET}", "s_nop 0",
        "buffer_load_dwordx4 %[slab_off], %[rsrc_as], %[slab_k] offen lds",
        "s_add_u32 m0, m0, 0x400", f"s_add_u32 {OFFSET}, %[slab_k], %[slab_rows]",
        f"buffer_load_dwordx4 %[slab_off], %[rsrc_as], {OFFSET} offen lds",
        f"s_mov_b32 m0, {W_TARGET}", "s_nop 0",
        "buffer_load_dword %[wslab_off], %[rsrc_ws], %[slab_k] offen lds",
        # the slab after this one: 32 bytes further along every row of scales, into the other buffers
        "s_add_u32 %[slab_k], %[slab_k], 32",
        f"s_xor_b32 {SLAB_TARGET}, {SLAB_TARGET}, 0x2000", f"s_xor_b32 {W_TARGET}, {W_TARGET}, 0x100",
    ]


def products(columns, split):
    """a_s * w_s of the next group for the given token tiles, rounded to FP32 (v_mul), set 0 with the
    wavefront's first scale block and, when its rows reach a second block, set 1 with that."""
    lines = []
    for j in columns:
        lines.append(f"v_mul_f32_e32 v{PROD + j}, v{NEXT_A + j}, v{NEXT_W}")
        if split < NA:
            lines.append(f"v_mul_f32_e32 v{PROD + 8 + j}, v{NEXT_A + j}, v{NEXT_W + 1}")
    return lines


def accumulate(tile, split):
    i, j = divmod(tile, NB)
    slot = DOT + 4 * (tile % 4)
    scale = PROD + (8 if i >= split else 0) + j
    base = 4 * tile
    return [f"v_fmac_f32_e32 v{base + r}, v{slot + r}, v{scale}" for r in range(4)]


DROP = set()  # experiments only: parts of a step left out (results are then wrong), see --drop
# a fill behind every FILL_EVERY-th matrix instruction of a step from FILL_FROM on (the fills are waited for
# at the end of the step they are issued in, so they go first: every third from the third on 514 us at 4096
# tokens, every second from the second on 489)
FILL_EVERY, FILL_FROM = 2, 1


def step(buffer, split, *, fills, reads, first, last, scale_step):
    """One K group: buffer = fragment buffer (and LDS stage) of this group. fills: LDS target of the
    group after the next, or None; reads: read the next group's fragments and scales; first: no tiles
    of a previous group are waiting for their accumulate; last: all 48 tiles are accumulated before
    the statement ends; scale_step: what the lane's slab address does after its reads
    ("next": the next group of the slab; "wrap": back to the slab's first group in the other buffer)."""
    units = fill_units(fills) if fills and "fills" not in DROP else []
    pending_reads = []
    if reads:
        pending_reads = ([] if "scales" in DROP else scale_reads()) + (
            [] if "reads" in DROP else fragment_reads(1 - buffer, 1 - buffer))
    lines = []
    fill_at = {FILL_EVERY * n + FILL_FROM: unit for n, unit in enumerate(units)}
    for t in range(TILES):
        i, j = divmod(t, NB)
        if t in fill_at:
            lines += fill_at[t][0]
        a, b = a_frag(buffer, i), b_frag(buffer, j)
        slot = DOT + 4 * (t % 4)
        lines.append(f"v_mfma_scale_f32_16x16x128_f8f6f4 v[{slot}:{slot + 3}], a[{a}:{a + 7}], a[{b}:{b + 7}], 0, "
                     f"v{UNIT}, v{UNIT} op_sel_hi:[0,0,0]")
        if t in fill_at:
            lines.append(fill_at[t][1])
            if fill_at[t] is units[-1]:
                lines += ADVANCE
        if "fmas" in DROP:
            pass
        elif t >= 2:
            lines += accumulate(t - 2, split)
        elif not first:  # the previous group's last two tiles, then the products they still needed
            lines += accumulate(TILES - 2 + t, split)
            lines += products([NB - 2 + t], split)
        if pending_reads and t < len(pending_reads):
            lines.append(pending_reads[t])
    assert len(pending_reads) <= TILES
    if reads:
        # the next group's products, except the two that the last two tiles' accumulates still use
        lines += ["s_waitcnt lgkmcnt(0)"] + products(range(NB - 2), split)
        if scale_step == "next":
            lines += ["v_add_u32_e32 %[sa], 4, %[sa]", "v_add_u32_e32 %[sw], 4, %[sw]"]
        else:  # eight groups on: the first group of the other slab buffers
            lines += ["v_subrev_u32_e32 %[sa], 28, %[sa]", "v_xor_b32_e32 %[sa], 0x2000, %[sa]",
                      "v_subrev_u32_e32 %[sw], 28, %[sw]", "v_xor_b32_e32 %[sw], 0x100, %[sw]"]
    if last:
        # (the results of the last two matrix instructions: more wait states than their latency)
        lines += ["s_nop 15", "s_nop 15"] + accumulate(TILES - 2, split) + accumulate(TILES - 1, split)
    else:
        lines += ["s_waitcnt lgkmcnt(0)" if "fillwait" in DROP else "s_waitcnt vmcnt(0) lgkmcnt(0)"]
        lines += [] if "barrier" in DROP else ["s_barrier"]
    return lines


def program(split):
    lines = [
        f"s_mov_b32 {SAVED_M0}, m0",
        f"s_add_u32 {FILL1}, %[fill0], {STAGE:#x}",
        f"v_mov_b32_e32 v{UNIT}, 0x7f7f7f7f",
        f"v_add_u32_e32 v{STAGE1}, {STAGE:#x}, %[ra_lo]", f"v_add_u32_e32 v{STAGE1 + 1}, {STAGE:#x}, %[ra_hi]",
        f"v_add_u32_e32 v{STAGE1 + 2}, {STAGE:#x}, %[rb_lo]", f"v_add_u32_e32 v{STAGE1 + 3}, {STAGE:#x}, %[rb_hi]",
        f"s_mov_b32 {SLAB_TARGET}, %[slab_fill]", f"s_mov_b32 {W_TARGET}, %[wslab_fill]",
    ]
    lines += [f"v_mov_b32_e32 v{r}, 0" for r in range(4 * TILES)]
    # slab 0 and group 0 into stage 0; then group 1 into stage 1, group 0's fragments and scales
    lines += ["; slab 0, group 0"] + slab_loads()
    for before, load in fill_units("%[fill0]"):
        lines += before + ["s_nop 0", load]
    lines += ADVANCE + ["s_waitcnt vmcnt(0)", "s_barrier", "; group 1 into stage 1"]
    for before, load in fill_units(FILL1):
        lines += before + ["s_nop 0", load]
    lines += ADVANCE + scale_reads() + fragment_reads(0, 0) + ["s_waitcnt lgkmcnt(0)"]
    lines += products(range(NB), split) + ["v_add_u32_e32 %[sa], 4, %[sa]", "v_add_u32_e32 %[sw], 4, %[sw]"]
    # every wavefront has read stage 0 and group 1 has landed before stage 0 is filled again and stage 1 is read
    lines += ["s_waitcnt vmcnt(0)", "s_barrier"]
    # A slab is eight steps, written out per position because the stage and the slab bookkeeping
    # repeat with periods 2 and 8 (fragment buffer = position % 2); its first step issues the next
    # slab's loads.
    def slab_steps(first_slab, last_slab):
        body = []
        for position in range(8):
            fills_target = None
            if not (last_slab and position >= 6):  # the group after the next exists
                fills_target = "%[fill0]" if position % 2 == 0 else FILL1
            reads = not (last_slab and position == 7)
            body.append(f"; slab position {position}")
            if position == 0 and not last_slab:
                body += slab_loads()
            body += step(position % 2, split, fills=fills_target, reads=reads,
                         first=first_slab and position == 0, last=last_slab and position == 7,
                         scale_step="wrap" if position == 6 else "next")
        return body

    # the first slab (no pending tiles at its start), the middle slabs in a loop, the last slab
    lines += ["; first slab"] + slab_steps(True, False)
    lines += ["s_cmp_eq_u32 %[middle], 0", "s_cbranch_scc1 L_fp8w4_last%=", "L_fp8w4_loop%=:"]
    lines += slab_steps(False, False)
    lines += ["s_sub_u32 %[middle], %[middle], 1", "s_cmp_lg_u32 %[middle], 0", "s_cbranch_scc1 L_fp8w4_loop%=",
              "L_fp8w4_last%=:"]
    lines += slab_steps(False, True)
    lines += [f"s_mov_b32 m0, {SAVED_M0}"]
    return lines


def statement(split):
    text = ["asm volatile("]
    for line in "\n".join(program(split)).split("\n"):
        text.append(f'    "{line}\\n"')
    outputs = [f'"=&{{{acc(*divmod(t, NB))}}}"(accs[{t}])' for t in range(TILES)]
    outputs += ['[a_off] "+v"(a_offset)', '[b_off] "+v"(b_offset)', '[sa] "+v"(scale_address)',
                '[sw] "+v"(weight_scale_address)', '[middle] "+s"(middle_slabs)', '[slab_k] "+s"(slab_k)']
    inputs = ['[ra_lo] "v"(read_a_lo)', '[ra_hi] "v"(read_a_hi)', '[rb_lo] "v"(read_b_lo)', '[rb_hi] "v"(read_b_hi)',
              '[slab_off] "v"(slab_offset)', '[wslab_off] "v"(weight_slab_offset)', '[rsrc_a] "s"(a_resource)',
              '[rsrc_b] "s"(b_resource)', '[rsrc_as] "s"(a_scale_resource)', '[rsrc_ws] "s"(w_scale_resource)',
              '[row_step] "s"(row_step)', '[fill0] "s"(fill_base)', '[slab_fill] "s"(slab_fill)',
              '[wslab_fill] "s"(weight_slab_fill)', '[slab_rows] "s"(slab_rows)']
    clobbers = ['"memory"', '"scc"'] + [f'"{s}"' for s in (SAVED_M0, OFFSET, FILL1, SLAB_TARGET, W_TARGET)]
    clobbers += [f'"v{n}"' for n in range(DOT, SCRATCH + 1)] + [f'"a{n}"' for n in range(2 * FRAG)]

    def wrapped(items):
        rows, row = [], "   "
        for item in items:
            if len(row) + len(item) > 108:
                rows.append(row)
                row = "   "
            row += " " + item + ","
        rows.append(row.rstrip(","))
        return rows

    text += ["    :"] + wrapped(outputs) + ["    :"] + wrapped(inputs) + ["    :"] + wrapped(clobbers) + [");"]
    return "\n".join(text)


def main():
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("--out", type=Path, default=Path(__file__).resolve().parent)
    parser.add_argument("--drop", default="", help="experiments: comma list of fills, reads, scales, fmas, barrier, fillwait")
    parser.add_argument("--placement", default="", help="experiments: FILL_EVERY,FILL_FROM")
    arguments = parser.parse_args()
    DROP.update(part for part in arguments.drop.split(",") if part)
    if arguments.placement:
        globals()["FILL_EVERY"], globals()["FILL_FROM"] = (int(v) for v in arguments.placement.split(","))
    text = ["// Generated by gen_fp8_wave4_loop.py; edit the generator, not this file.",
            "// split: the first of the wavefront's six 16-row weight tiles that lies in its second scale block"]
    for index, split in enumerate((2, 4, 6)):
        text.append(("if" if index == 0 else "} else if") + f" (split == {split}) {{" if split != 6 else "} else {")
        text.append(statement(split))
    text.append("}")
    (arguments.out / "fp8_wave4_loop_192x256.inc").write_text("\n".join(text) + "\n")


if __name__ == "__main__":
    main()
