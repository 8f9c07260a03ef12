#!/usr/bin/env python3
"""Writes mx_wave4_loop_192x256.inc: the K loop of mx_wave4.hip as one inline-assembly statement.

The E8M0 block-scaled prefill product (E4M3 inputs with one scale byte per 32 inputs, E4M3 weights with
one scale byte per 32 x 32 block) on four wavefronts per workgroup, one per SIMD: a workgroup owns 192
weight rows x 256 tokens, a wavefront 96 x 128 = 6 x 8 tiles of v_mfma_scale_f32_16x16x128_f8f6f4, one
instruction per tile and 128-input K group with the hardware applying both scales, so the accumulators are
touched by nothing but the matrix instructions.

The tile, the LDS stages and their fills, the fragment reads into accumulation registers and the slabs
through which scales reach the lanes are those of gen_fp8_wave4_loop.py (its functions are used here);
what differs is the scale handling. A lane group c = lane / 16 supplies the scale byte of inputs
32 c .. 32 c + 31 of its row; the four bytes of a row and K group are one 32-bit word of the slab, so a
lane reads its byte with ds_read_u8 at (word address + c) and the instruction takes byte 0 of the register.
Registers of a wavefront:
  v0..v191    the 48 accumulator tiles (C and D of the matrix instructions)
  v192..v213  two sets of eleven scale registers (eight token tiles; three weight registers, because a
              32-row scale block holds two 16-row tiles): the set of the group being multiplied and the
              set being read for the next group
  a0..a223    the operand fragments of two K groups
Usage: python gen_mx_wave4_loop.py [--out DIR]
"""

import argparse
from pathlib import Path

import gen_fp8_wave4_loop as base
from gen_fp8_wave4_loop import ADVANCE, FILL1, NA, NB, SAVED_M0, SLAB_TARGET, STAGE, STAGE1, TILES, W_TARGET

SCALES = 192  # first scale register; set s at SCALES + 11 s: tokens 0..7, then weight blocks 0..2
SET = NB + NA // 2


def scale_reads(into):
    """The next group's scale bytes: the lane's eight tokens (512 bytes apart in a slab of
    [token][8 groups] words) and the three 32-row blocks its 96 weight rows lie in (rows of 8 words)."""
    first = SCALES + SET * into
    lines = [f"ds_read_u8 v{first + j}, %[sa] offset:{512 * j}" for j in range(NB)]
    lines += [f"ds_read_u8 v{first + NB + b}, %[sw] offset:{32 * b}" for b in range(NA // 2)]
    return lines


def step(buffer, *, fills, reads, first, last, scale_step):
    """One K group from fragment buffer `buffer` with scale set `buffer`. fills: LDS target of the group
    after the next, or None; reads: fetch the next group's fragments and scales into the other buffer and
    set; first: the accumulators start from zero; scale_step as in gen_fp8_wave4_loop.step."""
    units = base.fill_units(fills) if fills else []
    pending = (scale_reads(1 - buffer) + base.fragment_reads(1 - buffer, 1 - buffer)) if reads else []
    assert len(pending) <= TILES
    fill_at = {3 * n + 2: unit for n, unit in enumerate(units)}
    scales = SCALES + SET * buffer
    lines = []
    for t in range(TILES):
        i, j = divmod(t, NB)
        if t in fill_at:
            lines += fill_at[t][0]
        a, b = base.a_frag(buffer, i), base.b_frag(buffer, j)
        acc = f"v[{4 * t}:{4 * t + 3}]"
        lines.append(f"v_mfma_scale_f32_16x16x128_f8f6f4 {acc}, a[{a}:{a + 7}], a[{b}:{b + 7}], {'0' if first else acc}, "
                     f"v{scales + NB + i // 2}, v{scales + j} op_sel_hi:[0,0,0]")
        if t in fill_at:
            lines.append(fill_at[t][1])
            if fill_at[t] is units[-1]:
                lines += ADVANCE
        if t < len(pending):
            lines.append(pending[t])
    if reads:
        if scale_step == "next":
            lines += ["v_add_u32_e32 %[sa], 4, %[sa]", "v_add_u32_e32 %[sw], 4, %[sw]"]
        else:  # eight groups on: the first group of the other slab buffers
            lines += ["v_subrev_u32_e32 %[sa], 28, %[sa]", "v_xor_b32_e32 %[sa], 0x2000, %[sa]",
                      "v_subrev_u32_e32 %[sw], 28, %[sw]", "v_xor_b32_e32 %[sw], 0x100, %[sw]"]
    if last:  # the code after the statement reads the accumulators: cover the longest instruction latency
        lines += ["s_nop 15", "s_nop 15"]
    else:
        lines += ["s_waitcnt vmcnt(0) lgkmcnt(0)", "s_barrier"]
    return lines


def program():
    lines = [
        f"s_mov_b32 {SAVED_M0}, m0",
        f"s_add_u32 {FILL1}, %[fill0], {STAGE:#x}",
        f"v_add_u32_e32 v{STAGE1}, {STAGE:#x}, %[ra_lo]", f"v_add_u32_e32 v{STAGE1 + 1}, {STAGE:#x}, %[ra_hi]",
        f"v_add_u32_e32 v{STAGE1 + 2}, {STAGE:#x}, %[rb_lo]", f"v_add_u32_e32 v{STAGE1 + 3}, {STAGE:#x}, %[rb_hi]",
        f"s_mov_b32 {SLAB_TARGET}, %[slab_fill]", f"s_mov_b32 {W_TARGET}, %[wslab_fill]",
        "; slab 0, group 0",
    ]
    lines += base.slab_loads()
    for before, load in base.fill_units("%[fill0]"):
        lines += before + ["s_nop 0", load]
    lines += ADVANCE + ["s_waitcnt vmcnt(0)", "s_barrier", "; group 1 into stage 1"]
    for before, load in base.fill_units(FILL1):
        lines += before + ["s_nop 0", load]
    lines += ADVANCE + scale_reads(0) + base.fragment_reads(0, 0)
    lines += ["v_add_u32_e32 %[sa], 4, %[sa]", "v_add_u32_e32 %[sw], 4, %[sw]"]
    # every wavefront has read stage 0 and group 1 has landed before stage 0 is filled again and stage 1 is read
    lines += ["s_waitcnt vmcnt(0) lgkmcnt(0)", "s_barrier"]

    def slab_steps(first_slab, last_slab):
        body = []
        for position in range(8):
            target = None
            if not (last_slab and position >= 6):
                target = "%[fill0]" if position % 2 == 0 else FILL1
            body.append(f"; slab position {position}")
            if position == 0 and not last_slab:
                body += base.slab_loads()
            body += step(position % 2, fills=target, reads=not (last_slab and position == 7),
                         first=first_slab and position == 0, last=last_slab and position == 7,
                         scale_step="wrap" if position == 6 else "next")
        return body

    lines += ["; first slab"] + slab_steps(True, False)
    lines += ["s_cmp_eq_u32 %[middle], 0", "s_cbranch_scc1 L_mxw4_last%=", "L_mxw4_loop%=:"]
    lines += slab_steps(False, False)
    lines += ["s_sub_u32 %[middle], %[middle], 1", "s_cmp_lg_u32 %[middle], 0", "s_cbranch_scc1 L_mxw4_loop%=",
              "L_mxw4_last%=:"]
    lines += slab_steps(False, True)
    lines += [f"s_mov_b32 m0, {SAVED_M0}"]
    return lines


def statement():
    text = ["// Generated by gen_mx_wave4_loop.py; edit the generator, not this file.", "asm volatile("]
    for line in "\n".join(program()).split("\n"):
        text.append(f'    "{line}\\n"')
    outputs = [f'"=&{{{base.acc(*divmod(t, NB))}}}"(accs[{t}])' for t in range(TILES)]
    outputs += ['[a_off] "+v"(a_offset)', '[b_off] "+v"(b_offset)', '[sa] "+v"(scale_address)',
                '[sw] "+v"(weight_scale_address)', '[middle] "+s"(middle_slabs)', '[slab_k] "+s"(slab_k)']
    inputs = ['[ra_lo] "v"(read_a_lo)', '[ra_hi] "v"(read_a_hi)', '[rb_lo] "v"(read_b_lo)', '[rb_hi] "v"(read_b_hi)',
              '[slab_off] "v"(slab_offset)', '[wslab_off] "v"(weight_slab_offset)', '[rsrc_a] "s"(a_resource)',
              '[rsrc_b] "s"(b_resource)', '[rsrc_as] "s"(a_scale_resource)', '[rsrc_ws] "s"(w_scale_resource)',
              '[row_step] "s"(row_step)', '[fill0] "s"(fill_base)', '[slab_fill] "s"(slab_fill)',
              '[wslab_fill] "s"(weight_slab_fill)', '[slab_rows] "s"(slab_rows)']
    clobbers = ['"memory"', '"scc"'] + [f'"{s}"' for s in (SAVED_M0, base.OFFSET, FILL1, SLAB_TARGET, W_TARGET)]
    clobbers += [f'"v{n}"' for n in range(SCALES, SCALES + 2 * SET)]
    clobbers += [f'"v{n}"' for n in range(STAGE1, STAGE1 + 4)] + [f'"a{n}"' for n in range(2 * base.FRAG)]

    def wrapped(items):
        rows, row = [], "   "
        for item in items:
            if len(row) + len(item) > 108:
                rows.append(row)
                row = "   "
            row += " " + item + ","
        rows.append(row.rstrip(","))
        return rows

    text += ["    :"] + wrapped(outputs) + ["    :"] + wrapped(inputs) + ["    :"] + wrapped(clobbers) + [");", ""]
    return "\n".join(text)


def main():
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("--out", type=Path, default=Path(__file__).resolve().parent)
    arguments = parser.parse_args()
    (arguments.out / "mx_wave4_loop_192x256.inc").write_text(statement())


if __name__ == "__main__":
    main()
