#!/usr/bin/env python3
"""Writes mx_wave4_loop_192x256.inc and mx_wave4_loop_192x256_e2m1.inc: the K loops of mx_wave4.hip, each
one inline-assembly statement.

The E8M0 block-scaled prefill product (E4M3 inputs with one scale byte per 32 inputs; E4M3 weights with
one scale byte per 32 x 32 block, or packed E2M1 weights with one scale byte per row and 32 inputs) on
four wavefronts per workgroup, one per SIMD: a workgroup owns 192 weight rows x 256 tokens, a wavefront
96 x 128 = 6 x 8 tiles of v_mfma_scale_f32_16x16x128_f8f6f4, one instruction per tile and 128-input K
group with the hardware applying both scales, so the accumulators are touched by nothing but the matrix
instructions.

One K group (step) of a wavefront: 48 matrix instructions back to back on the fragments and scale bytes
of this group; spread between them the LDS reads of the next group's scale bytes and fragments into the
other register sets, and the direct-to-LDS fills of the group after that into the LDS stage the next
group's fragments are NOT in (this group's, whose fragments were read a step ago). One wait and one
barrier per group. Every eighth group the next eight groups' scale words (four scale bytes of a row and
group) are copied into LDS slabs, 16 bytes per lane (4 bytes for the block rows of E4M3 weights).

Scale bytes: lane group c = lane / 16 supplies the scale of inputs 32 c .. 32 c + 31 of its row, so a
lane reads its byte with ds_read_u8 at (word address + c) and the instruction takes byte 0 of the register.
Registers of a wavefront:
  v0..v191     the 48 accumulator tiles (C and D of the matrix instructions)
  v192..       two sets of scale registers, eight token tiles and the weight tiles' (E4M3 weights: three,
               a 32-row block holds two 16-row tiles; E2M1: six): the set of the group being multiplied
               and the set being read for the next group
  v235..v238   LDS read addresses of stage 1
  a0..         the operand fragments of two K groups (an E4M3 fragment is eight registers: the 16 bytes at
               chunk c and at chunk 4 + c of the lane's 128-byte row; an E2M1 fragment four: chunk c of the
               lane's 64-byte row)
The fragment files use local variables of the including function by name (see mx_wave4.hip).
Usage: python gen_mx_wave4_loop.py [--out DIR]
"""

import argparse
from pathlib import Path

NA, NB = 6, 8  # 16-row weight tiles and 16-token tiles per wavefront
TILES = NA * NB
SCALES, STAGE1 = 192, 235
SAVED_M0, OFFSET, FILL1, SLAB_TARGET, W_TARGET = "s84", "s85", "s86", "s87", "s88"
# placement inside a step: a fill behind every FILL_EVERY-th matrix instruction from FILL_FROM on, an LDS read
# behind every instruction from READ_FROM on. The fills are waited for at the end of the step they are issued
# in, so they go first (measured, E4M3 weights at 4096 rows: fills every third instruction from the third on
# and reads from the first 418 us; fills every second from the first 396-400 us wherever the reads start; all
# fills in a burst 417 us)
FILL_EVERY, FILL_FROM, READ_FROM = 2, 0, 8


class Form:
    def __init__(self, packed):
        self.packed = packed
        self.a_regs = 4 if packed else 8  # registers of a weight fragment
        self.a_row = 64 if packed else 128  # bytes of a weight row in a K group
        self.a_bytes = 32 * NA * self.a_row  # weight rows of a stage
        self.a_fills = self.a_bytes // 4096  # 1 KB loads per wavefront
        self.stage = self.a_bytes + 256 * 128
        self.frag = self.a_regs * NA + 8 * NB  # accumulation registers of one fragment buffer
        self.w_scales = NA if packed else NA // 2
        self.set = NB + self.w_scales
        # the loop flips between the two buffers of a slab with one address bit
        self.w_flip = 0x2000 if packed else 0x100
        self.name = "mx_wave4_loop_192x256" + ("_e2m1" if packed else "") + ".inc"

    def a_frag(self, buffer, i):
        return buffer * self.frag + self.a_regs * i

    def b_frag(self, buffer, j):
        return buffer * self.frag + self.a_regs * NA + 8 * j

    def fragment_reads(self, stage, buffer):
        if stage == 0:
            names = ("%[ra_lo]", "%[ra_hi]", "%[rb_lo]", "%[rb_hi]")
        else:
            names = tuple(f"v{STAGE1 + n}" for n in range(4))
        lines = []
        for i in range(NA):
            r = self.a_frag(buffer, i)
            lines.append(f"ds_read_b128 a[{r}:{r + 3}], {names[0]} offset:{i * 16 * self.a_row}")
            if not self.packed:
                lines.append(f"ds_read_b128 a[{r + 4}:{r + 7}], {names[1]} offset:{i * 2048}")
        for j in range(NB):
            r = self.b_frag(buffer, j)
            lines.append(f"ds_read_b128 a[{r}:{r + 3}], {names[2]} offset:{j * 2048}")
            lines.append(f"ds_read_b128 a[{r + 4}:{r + 7}], {names[3]} offset:{j * 2048}")
        return lines

    def scale_reads(self, into):
        """The next group's scale bytes: the lane's eight tokens and its weight tiles' (E2M1: six rows in a
        slab of the tokens' shape; E4M3: the three 32-row blocks its 96 rows lie in, rows of 9 words: its
        32 scale bytes from wherever they lie after the aligned address the row was copied from). A slab
        of rows is pieces of 32 rows, a piece two halves (groups 0-3, groups 4-7) of [row][4 words]: sixteen
        rows in a row are sixteen different banks; rows 16 apart are 256 bytes apart, 32 apart a piece."""
        first = SCALES + self.set * into
        rows = lambda index: (index // 2) * 1024 + (index % 2) * 256
        lines = [f"ds_read_u8 v{first + j}, %[sa] offset:{rows(j)}" for j in range(NB)]
        lines += [f"ds_read_u8 v{first + NB + b}, %[sw] offset:{rows(b) if self.packed else 36 * b}"
                  for b in range(self.w_scales)]
        return lines

    def scale_advance(self, position):
        """What the lane's slab addresses do after the reads of the step at `position` of a slab (which read
        group position + 1): on to the next group's word: 4 bytes, from group 3 to group 4 into the piece's
        second half, from group 7 to group 0 of the other buffer."""
        rows = {2: ["v_add_u32_e32 {0}, 500, {0}"], 6: ["v_subrev_u32_e32 {0}, 524, {0}", "v_xor_b32_e32 {0}, 0x2000, {0}"]}
        blocks = {6: ["v_subrev_u32_e32 {0}, 28, {0}", "v_xor_b32_e32 {0}, 0x100, {0}"]}
        step = ["v_add_u32_e32 {0}, 4, {0}"]
        lines = [line.format("%[sa]") for line in rows.get(position, step)]
        lines += [line.format("%[sw]") for line in (rows if self.packed else blocks).get(position, step)]
        return lines

    def fill_units(self, target):
        """Per direct-to-LDS load: (scalar set-up, the load). M0 walks the wavefront's LDS slots in 4 KB
        strides through the weight rows and on into the token rows; the row advance of successive loads
        is the scalar offset."""
        units = []
        for n in range(self.a_fills + NB):
            weights = n < self.a_fills
            first = n == 0 or n == self.a_fills
            second = n == 1 or n == self.a_fills + 1
            lane, resource, step = (("%[a_off]", "%[rsrc_a]", "%[row_step_a]") if weights
                                    else ("%[b_off]", "%[rsrc_b]", "%[row_step]"))
            before = [f"s_mov_b32 m0, {target}" if n == 0 else "s_add_u32 m0, m0, 0x1000"]
            if second:
                before.append(f"s_mov_b32 {OFFSET}, {step}")
            elif not first:
                before.append(f"s_add_u32 {OFFSET}, {OFFSET}, {step}")
            units.append((before, f"buffer_load_dwordx4 {lane}, {resource}, {'0' if first else OFFSET} offen lds"))
        return units

    def advance(self):
        return [f"v_add_u32_e32 %[a_off], {self.a_row:#x}, %[a_off]", "v_add_u32_e32 %[b_off], 0x80, %[b_off]"]

    def slab_loads(self):
        """The next eight groups' scale words into the slab buffers that are not being read: two pieces of
        the token slab per wavefront (32 tokens each, lane l brings groups 4 (l / 32) .. + 3 of token
        l % 32); the weights' likewise (E2M1: pieces w and w + 4 of eight, of which six hold the tile's
        rows) or with one 4-byte-per-lane load (E4M3: every wavefront brings the same bytes to the same place)."""
        lines = [
            f"s_mov_b32 m0, {SLAB_TARGET}", "s_nop 0",
            "buffer_load_dwordx4 %[slab_off], %[rsrc_as], %[slab_k] offen lds",
            "s_add_u32 m0, m0, 0x400", f"s_add_u32 {OFFSET}, %[slab_k], %[slab_rows]",
            f"buffer_load_dwordx4 %[slab_off], %[rsrc_as], {OFFSET} offen lds",
            f"s_mov_b32 m0, {W_TARGET}", "s_nop 0",
        ]
        if self.packed:
            lines += ["buffer_load_dwordx4 %[wslab_off], %[rsrc_ws], %[slab_k] offen lds",
                      "s_add_u32 m0, m0, 0x1000", f"s_add_u32 {OFFSET}, %[slab_k], %[wslab_rows]",
                      f"buffer_load_dwordx4 %[wslab_off], %[rsrc_ws], {OFFSET} offen lds"]
        else:
            lines += ["buffer_load_dword %[wslab_off], %[rsrc_ws], %[slab_k] offen lds"]
        # the slab after this one: 32 bytes further along every row of scale words, into the other buffers
        lines += ["s_add_u32 %[slab_k], %[slab_k], 32", f"s_xor_b32 {SLAB_TARGET}, {SLAB_TARGET}, 0x2000",
                  f"s_xor_b32 {W_TARGET}, {W_TARGET}, {self.w_flip:#x}"]
        return lines

    def step(self, buffer, *, fills, reads, first, last, position):
        """One K group from fragment buffer `buffer` with scale set `buffer`. fills: LDS target of the group
        after the next, or None; reads: fetch the next group's fragments and scales into the other buffer
        and set; first: the accumulators start from zero; position: of the step in its slab."""
        units = self.fill_units(fills) if fills else []
        pending = (self.scale_reads(1 - buffer) + self.fragment_reads(1 - buffer, 1 - buffer)) if reads else []
        assert len(pending) + READ_FROM <= TILES and FILL_EVERY * len(units) <= TILES
        fill_at = {FILL_EVERY * n + FILL_FROM: unit for n, unit in enumerate(units)}
        scales = SCALES + self.set * buffer
        lines = []
        for t in range(TILES):
            i, j = divmod(t, NB)
            if t in fill_at:
                lines += fill_at[t][0]
            a, b = self.a_frag(buffer, i), self.b_frag(buffer, j)
            acc = f"v[{4 * t}:{4 * t + 3}]"
            weight_scale = scales + NB + (i if self.packed else i // 2)
            lines.append(f"v_mfma_scale_f32_16x16x128_f8f6f4 {acc}, a[{a}:{a + self.a_regs - 1}], a[{b}:{b + 7}], "
                         f"{'0' if first else acc}, v{weight_scale}, v{scales + j} op_sel_hi:[0,0,0]"
                         + (" cbsz:4" if self.packed else ""))
            if t in fill_at:
                lines.append(fill_at[t][1])
                if fill_at[t] is units[-1]:
                    lines += self.advance()
            if 0 <= t - READ_FROM < len(pending):
                lines.append(pending[t - READ_FROM])
        if reads:
            lines += self.scale_advance(position)
        if last:  # the code after the statement reads the accumulators: cover the longest instruction latency
            lines += ["s_nop 15", "s_nop 15"]
        else:
            lines += ["s_waitcnt vmcnt(0) lgkmcnt(0)", "s_barrier"]
        return lines

    def program(self):
        lines = [
            f"s_mov_b32 {SAVED_M0}, m0",
            f"s_add_u32 {FILL1}, %[fill0], {self.stage:#x}",
            f"v_add_u32_e32 v{STAGE1}, {self.stage:#x}, %[ra_lo]", f"v_add_u32_e32 v{STAGE1 + 1}, {self.stage:#x}, %[ra_hi]",
            f"v_add_u32_e32 v{STAGE1 + 2}, {self.stage:#x}, %[rb_lo]", f"v_add_u32_e32 v{STAGE1 + 3}, {self.stage:#x}, %[rb_hi]",
            f"s_mov_b32 {SLAB_TARGET}, %[slab_fill]", f"s_mov_b32 {W_TARGET}, %[wslab_fill]",
            "; slab 0, group 0",
        ]
        lines += self.slab_loads()
        for before, load in self.fill_units("%[fill0]"):
            lines += before + ["s_nop 0", load]
        lines += self.advance() + ["s_waitcnt vmcnt(0)", "s_barrier", "; group 1 into stage 1"]
        for before, load in self.fill_units(FILL1):
            lines += before + ["s_nop 0", load]
        lines += self.advance() + self.scale_reads(0) + self.fragment_reads(0, 0) + self.scale_advance(7)
        # every wavefront has read stage 0 and group 1 has landed before stage 0 is filled again and stage 1 is read
        lines += ["s_waitcnt vmcnt(0) lgkmcnt(0)", "s_barrier"]

        def slab_steps(first_slab, last_slab):
            # a slab is eight steps, written out per position because the stage and the slab bookkeeping
            # repeat with periods 2 and 8; its first step issues the next slab's loads
            body = []
            for position in range(8):
                target = None
                if not (last_slab and position >= 6):
                    target = "%[fill0]" if position % 2 == 0 else FILL1
                body.append(f"; slab position {position}")
                if position == 0 and not last_slab:
                    body += self.slab_loads()
                body += self.step(position % 2, fills=target, reads=not (last_slab and position == 7),
                                  first=first_slab and position == 0, last=last_slab and position == 7,
                                  position=position)
            return body

        lines += ["; first slab"] + slab_steps(True, False)
        lines += ["s_cmp_eq_u32 %[middle], 0", "s_cbranch_scc1 L_mxw4_last%=", "L_mxw4_loop%=:"]
        lines += slab_steps(False, False)
        lines += ["s_sub_u32 %[middle], %[middle], 1", "s_cmp_lg_u32 %[middle], 0", "s_cbranch_scc1 L_mxw4_loop%=",
                  "L_mxw4_last%=:"]
        lines += slab_steps(False, True)
        lines += [f"s_mov_b32 m0, {SAVED_M0}"]
        return lines

    def statement(self):
        text = ["// Generated by gen_mx_wave4_loop.py; edit the generator, not this file.", "asm volatile("]
        for line in "\n".join(self.program()).split("\n"):
            text.append(f'    "{line}\\n"')
        outputs = [f'"=&{{v[{4 * t}:{4 * t + 3}]}}"(accs[{t}])' for t in range(TILES)]
        outputs += ['[a_off] "+v"(a_offset)', '[b_off] "+v"(b_offset)', '[sa] "+v"(scale_address)',
                    '[sw] "+v"(weight_scale_address)', '[middle] "+s"(middle_slabs)', '[slab_k] "+s"(slab_k)']
        inputs = ['[ra_lo] "v"(read_a_lo)', '[ra_hi] "v"(read_a_hi)', '[rb_lo] "v"(read_b_lo)', '[rb_hi] "v"(read_b_hi)',
                  '[slab_off] "v"(slab_offset)', '[wslab_off] "v"(weight_slab_offset)', '[rsrc_a] "s"(a_resource)',
                  '[rsrc_b] "s"(b_resource)', '[rsrc_as] "s"(a_scale_resource)', '[rsrc_ws] "s"(w_scale_resource)',
                  '[row_step] "s"(row_step)', '[row_step_a] "s"(row_step_a)', '[fill0] "s"(fill_base)',
                  '[slab_fill] "s"(slab_fill)', '[wslab_fill] "s"(weight_slab_fill)', '[slab_rows] "s"(slab_rows)',
                  '[wslab_rows] "s"(weight_slab_rows)']
        clobbers = ['"memory"', '"scc"'] + [f'"{s}"' for s in (SAVED_M0, OFFSET, FILL1, SLAB_TARGET, W_TARGET)]
        clobbers += [f'"v{n}"' for n in range(SCALES, SCALES + 2 * self.set)]
        clobbers += [f'"v{n}"' for n in range(STAGE1, STAGE1 + 4)] + [f'"a{n}"' for n in range(2 * self.frag)]

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
    parser.add_argument("--placement", default="", help="experiments: FILL_EVERY,FILL_FROM,READ_FROM")
    arguments = parser.parse_args()
    if arguments.placement:
        globals()["FILL_EVERY"], globals()["FILL_FROM"], globals()["READ_FROM"] = (int(v) for v in arguments.placement.split(","))
    for packed in (False, True):
        form = Form(packed)
        (arguments.out / form.name).write_text(form.statement())


if __name__ == "__main__":
    main()
