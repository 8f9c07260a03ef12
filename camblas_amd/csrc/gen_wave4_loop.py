#!/usr/bin/env python3
"""Writes wave4_loop_<rows>x256.inc: the K loop of bgemm_wave4.hip as one inline-assembly statement.

Why the loop is generated assembly and not HIP source: a workgroup of four wavefronts, one per SIMD,
each owning a (16*NA) x 128 block of the output tile, keeps 4*NA*8 FP32 accumulators per lane. They
fill the accumulation half of the register file (a0..a255; what does not fit goes to named
architectural registers), and the operand fragments, double-buffered per 32-deep sub-step, take the
low architectural registers. The compiler's allocator spreads such a kernel over both halves and
spills; with every register named here it has nothing to decide inside the loop.

One K step (64 elements) of a wavefront:
  phase 1  NA*8 matrix instructions on fragment buffer 1 (second sub-step of the previous K step)
           | direct-to-LDS fills of the K step after this one | LDS reads of this step's first
           sub-step into buffer 0
  phase 2  NA*8 matrix instructions on buffer 0 | LDS reads of the second sub-step into buffer 1
  wait for the fills and the reads, barrier
so the matrix pipe always has a full sub-step of independent instructions while the next operands
travel, and the only point where the four wavefronts meet is one barrier per K step.

The fragment file uses local variables of the including function by name: accs[] (f32x4_t outputs, tile (i, j) at 8 i + j),
a_offset / b_offset (per-lane byte offsets of the fills, advanced by the loop), read_a0 / read_a1 /
read_b0 / read_b1 (LDS byte addresses of the first weight / token fragment for sub-step 0 / 1 in
stage 0), a_resource / b_resource (u32x4_t buffer descriptors), a_row_step / b_row_step (bytes
between successive fill rows), fill_base (this wavefront's first LDS fill address in stage 0) and
step_pairs ((K steps - 2) / 2).

Usage: python gen_wave4_loop.py [--out DIR] [--drop fills,barrier,fillwait,reads]
Without arguments it rewrites the .inc files beside this script. --drop leaves mechanisms out of the
loop for timing-only builds that attribute the kernel's time (their results are wrong by design;
such files are written somewhere else with --out and never shipped).
"""

import argparse
from pathlib import Path

DROP = set()

NB = 8  # token tiles of 16 per wavefront: 128 tokens, two wavefronts across = 256


NN_PIECE = 1056  # bytes from one 1 KB piece of an as-it-lies weight tile to the next (see Layout)


class Layout:
    """na: 16-row weight tiles per wavefront. nn: the weights lie the other way round, K rows of
    contiguous outputs (x @ W with a row-major W). A K step of such a tile is 64 rows of 512 bytes;
    a direct-to-LDS load brings rows k and k + 4 (1 KB), pieces are placed 1056 bytes apart, and a lane
    gathers its eight K values of one output with two ds_read_b64_tr_b16: within sixteen lanes, lane
    4a + b receives element b of the four values at the addresses of lanes a, 4 + a, 8 + a, 12 + a,
    so lane s points at row s / 4 of a four-row group, outputs 4 (s % 4) .. + 3, and receives four
    K values of output s. The four rows of a group lie in four different pieces and the second group
    of a 32-lane half (rows + 8) in four more: eight 32-byte runs in eight different bank windows."""

    def __init__(self, na, nn=False):
        self.na = na
        self.nn = nn
        self.rows = 32 * na  # weight rows of the workgroup tile (two wavefronts down)
        assert not nn or na == 8, "a K row of 256 outputs is half a 1 KB load"
        self.a_bytes = 32 * NN_PIECE if nn else self.rows * 128
        self.stage_bytes = self.a_bytes + 256 * 128
        self.frag = 4 * (na + NB)  # registers of one fragment buffer
        self.buffers = (0, self.frag)
        # accumulators beyond a0..a255 live in architectural registers behind the fragment buffers
        self.extra_acc_base = 2 * self.frag
        self.extra_acc = max(0, 4 * na * NB - 256)
        self.scratch_v = self.extra_acc_base + self.extra_acc  # four stage-1 read addresses
        self.clobbered_v = self.scratch_v + 4

    def a_frag(self, buffer, i):
        return self.buffers[buffer] + 4 * i

    def b_frag(self, buffer, j):
        return self.buffers[buffer] + 4 * (self.na + j)

    def acc(self, i, j):
        index = 4 * (i * NB + j)
        if index < 256:
            return f"a[{index}:{index + 3}]"
        index = self.extra_acc_base + index - 256
        return f"v[{index}:{index + 3}]"


SAVED_M0, OFFSET, FILL1, FILL1B = "s84", "s85", "s86", "s87"


def fill_units(layout, target, target_b=None):
    """Per direct-to-LDS load: (scalar set-up placed before a matrix instruction, the load after it).
    M0 walks this wavefront's LDS slots in 4 KB strides through the weight rows and on into the
    token rows; the row advance of successive loads is the scalar offset. (As-it-lies weights: the
    wavefront's pieces are four pieces, 4224 bytes, apart, and the token rows start at target_b.)"""
    units = []
    for n in range(layout.na + NB):
        weights = n < layout.na
        first = n == 0 or n == layout.na
        second = n == 1 or n == layout.na + 1
        lane, resource, step = (("%[a_off]", "%[rsrc_a]", "%[a_step]") if weights
                                else ("%[b_off]", "%[rsrc_b]", "%[b_step]"))
        if n == 0:
            before = [f"s_mov_b32 m0, {target}"]
        elif layout.nn and n == layout.na:
            before = [f"s_mov_b32 m0, {target_b}"]
        else:
            before = [f"s_add_u32 m0, m0, {4 * NN_PIECE:#x}" if layout.nn and weights else "s_add_u32 m0, m0, 0x1000"]
        if second:
            before.append(f"s_mov_b32 {OFFSET}, {step}")
        elif not first:
            before.append(f"s_add_u32 {OFFSET}, {OFFSET}, {step}")
        load = f"buffer_load_dwordx4 {lane}, {resource}, {'0' if first else OFFSET} offen lds"
        if "fills" in DROP:
            load = "s_nop 0"
        # timing experiments: the same bytes fetched into registers instead of LDS, and / or written
        # to LDS from registers
        stage = layout.clobbered_v + 4 * n
        offset = n * 4096
        to_register = f"buffer_load_dwordx4 v[{stage}:{stage + 3}], {lane}, {resource}, {'0' if first else OFFSET} offen"
        write = f"ds_write_b128 %[ra0], v[{stage}:{stage + 3}] offset:{offset}"
        if "tovgpr" in DROP:
            load = to_register
        if "dswrite" in DROP:
            load = write
        if "staged" in DROP:
            load = write + "\n" + to_register
        units.append((before, load))
    return units


def advance(layout):
    """The fills' per-lane offsets move on by one K step: 64 elements along a K-contiguous row, 64 rows
    of an as-it-lies weight matrix."""
    weights = "v_add_u32_e32 %[a_off], %[a_kstep], %[a_off]" if layout.nn else "v_add_u32_e32 %[a_off], 0x80, %[a_off]"
    return [weights, "v_add_u32_e32 %[b_off], 0x80, %[b_off]"]


def reads(layout, stage, sub_step, buffer):
    """LDS reads of one sub-step's fragments: weight fragments first, token fragments after (the
    token fragments of the buffer being overwritten are the last the previous phase still uses)."""
    if stage == 0:
        a_address, b_address = f"%[ra{sub_step}]", f"%[rb{sub_step}]"
    else:
        a_address = f"v{layout.scratch_v + sub_step}"
        b_address = f"v{layout.scratch_v + 2 + sub_step}"
    lines = []
    for i in range(layout.na):
        r = layout.a_frag(buffer, i)
        if layout.nn:
            # K values 8 q .. + 3 and + 4 .. + 7 of the sub-step for lane group q: rows four apart are the
            # two halves of a piece, a sub-step is sixteen pieces, the next sixteen outputs 32 bytes on
            address = "%[ra0]" if stage == 0 else f"v{layout.scratch_v}"
            offset = sub_step * 16 * NN_PIECE + i * 32
            lines.append(f"ds_read_b64_tr_b16 v[{r}:{r + 1}], {address} offset:{offset}")
            lines.append(f"ds_read_b64_tr_b16 v[{r + 2}:{r + 3}], {address} offset:{offset + 512}")
        else:
            lines.append(f"ds_read_b128 v[{r}:{r + 3}], {a_address} offset:{i * 2048}")
    for j in range(NB):
        r = layout.b_frag(buffer, j)
        lines.append(f"ds_read_b128 v[{r}:{r + 3}], {b_address} offset:{j * 2048}")
    if "reads" in DROP:
        return []
    return lines


FILL_EVERY = 4  # a fill after every FILL_EVERY-th matrix instruction
ORDER = "weights"  # consecutive matrix instructions share their weight fragment ("tokens", "snake": experiments)


def tile_order(layout):
    if ORDER == "tokens":
        return [(i, j) for j in range(NB) for i in range(layout.na)]
    if ORDER == "snake":
        return [(i, j if i % 2 == 0 else NB - 1 - j) for i in range(layout.na) for j in range(NB)]
    return [(i, j) for i in range(layout.na) for j in range(NB)]


READS = "early"  # "late": an experiment, see k_step


class LdsQueue:
    """Counts this wavefront's LDS reads in issue order (they return in that order), so that a wait
    for one of them can leave the later ones outstanding: s_waitcnt lgkmcnt(n) with n = reads
    issued after it (the counter holds four bits)."""

    def __init__(self):
        self.issued = 0
        self.sequence = {}

    def issue(self, line):
        self.sequence[line.split(",")[0]] = self.issued  # keyed by destination registers
        self.issued += 1
        return line

    def wait_for(self, destination):
        return f"s_waitcnt lgkmcnt({min(15, self.issued - self.sequence[destination] - 1)})"


def phase(layout, buffer, read_lines, fills, zero=False, advance=False, read_every=2, queue=None, waits=False):
    """NA*8 matrix instructions on one fragment buffer with the fills and LDS reads between them:
    a fill after every FILL_EVERY-th instruction, a read after every read_every-th one, until both
    run out. waits: this buffer's fragments may still be on their way; wait for each weight
    fragment before its first use (the token fragments were requested before all of them)."""
    lines = []
    count = layout.na * NB
    fills = fills or []
    assert len(fills) <= (count + FILL_EVERY - 1) // FILL_EVERY and len(read_lines) * read_every <= count, (
        len(fills), len(read_lines), read_every, count)
    for k, (i, j) in enumerate(tile_order(layout)):
        unit = fills[k // FILL_EVERY] if k % FILL_EVERY == 0 and k // FILL_EVERY < len(fills) else None
        if unit:
            lines += unit[0]
        a, b = layout.a_frag(buffer, i), layout.b_frag(buffer, j)
        if waits and j == 0:
            lines.append(queue.wait_for(f"ds_read_b128 v[{a}:{a + 3}]"))
        source = "0" if zero else layout.acc(i, j)
        lines.append(f"v_mfma_f32_16x16x32_bf16 {layout.acc(i, j)}, v[{a}:{a + 3}], v[{b}:{b + 3}], {source}")
        if unit:
            lines.append(unit[1])
            if advance and unit is fills[-1]:
                lines += globals()["advance"](layout)
        if k % read_every == read_every - 1 and k // read_every < len(read_lines):
            line = read_lines[k // read_every]
            lines.append(queue.issue(line) if queue else line)
    return lines


def k_step(layout, stage, fill_target, fill_target_b=None):
    fills = fill_units(layout, fill_target, fill_target_b) if fill_target else []
    count = layout.na * NB
    first = min(len(fills), (count + FILL_EVERY - 1) // FILL_EVERY)
    lines = [f"; K step in stage {stage}" + (f", fills into {fill_target}" if fill_target else ", no fills")]
    first_reads, second_reads = reads(layout, stage, 0, 0), reads(layout, stage, 1, 1)
    if READS == "late" and first_reads:
        # the first sub-step's fragments are requested over the whole of phase 1, token fragments
        # first, and phase 2 waits for each weight fragment where it first needs it; phase 2's own
        # requests are spread over its first three quarters (they must be back before the barrier)
        queue = LdsQueue()
        first_reads = first_reads[layout.na:] + first_reads[:layout.na]
        lines += phase(layout, 1, first_reads, fills[:first], advance=first == len(fills),
                       read_every=count // len(first_reads), queue=queue)
        lines += phase(layout, 0, second_reads, fills[first:], advance=first < len(fills),
                       read_every=max(2, (3 * count // 4) // len(second_reads)), queue=queue, waits=True)
    else:
        lines += phase(layout, 1, first_reads, fills[:first], advance=first == len(fills))
        lines.append("s_waitcnt lgkmcnt(0)")
        lines += phase(layout, 0, second_reads, fills[first:], advance=first < len(fills))
    lines += ["s_waitcnt lgkmcnt(0)" if "fillwait" in DROP else "s_waitcnt vmcnt(0) lgkmcnt(0)"]
    if "barrier" not in DROP:
        lines.append("s_barrier")
    return lines


def program(layout):
    v = layout.scratch_v
    lines = [
        f"s_mov_b32 {SAVED_M0}, m0",
        f"s_add_u32 {FILL1}, %[fill0], {layout.stage_bytes:#x}",
        f"v_add_u32_e32 v{v}, {layout.stage_bytes:#x}, %[ra0]",
        f"v_add_u32_e32 v{v + 1}, {layout.stage_bytes:#x}, %[ra1]",
        f"v_add_u32_e32 v{v + 2}, {layout.stage_bytes:#x}, %[rb0]",
        f"v_add_u32_e32 v{v + 3}, {layout.stage_bytes:#x}, %[rb1]",
        "; K step 0 into stage 0",
    ]
    if layout.nn:
        lines.insert(2, f"s_add_u32 {FILL1B}, %[fill0b], {layout.stage_bytes:#x}")
    for before, load in fill_units(layout, "%[fill0]", "%[fill0b]"):
        lines += before + ["s_nop 0", load]
    lines += advance(layout) + ["s_waitcnt vmcnt(0)", "s_barrier", "; K step 1 into stage 1, first fragments of step 0"]
    for before, load in fill_units(layout, FILL1, FILL1B):
        lines += before + ["s_nop 0", load]
    lines += advance(layout) + reads(layout, 0, 0, 0) + ["s_waitcnt lgkmcnt(0)"]
    lines += phase(layout, 0, reads(layout, 0, 1, 1), None, zero=True)
    lines += ["s_waitcnt vmcnt(0) lgkmcnt(0)", "s_barrier",
              "s_cmp_eq_u32 %[pairs], 0", "s_cbranch_scc1 L_wave4_last%=", "L_wave4_loop%=:"]
    lines += k_step(layout, 1, "%[fill0]", "%[fill0b]")
    lines += k_step(layout, 0, FILL1, FILL1B)
    lines += ["s_sub_u32 %[pairs], %[pairs], 1", "s_cmp_lg_u32 %[pairs], 0", "s_cbranch_scc1 L_wave4_loop%=",
              "L_wave4_last%=:"]
    lines += k_step(layout, 1, None)
    lines += ["; second sub-step of the last K step"]
    lines += phase(layout, 1, [], None)
    # the code after this statement reads accumulators: cover the longest matrix-instruction latency
    lines += [f"s_mov_b32 m0, {SAVED_M0}", "s_nop 15", "s_nop 15"]
    return lines


def statement(layout):
    text = ["// Generated by gen_wave4_loop.py; edit the generator, not this file.", "asm volatile("]
    for line in "\n".join(program(layout)).split("\n"):
        text.append(f'    "{line}\\n"')
    # one four-wide output per accumulator tile (wider tuples of named accumulation registers trip the
    # compiler when single elements are taken from them)
    outputs = []
    for t in range(layout.na * NB):
        register = layout.acc(*divmod(t, NB))
        # (accumulators in architectural registers are marked early-clobber: without it the compiler
        # may hand the same registers to inputs, which the loop still reads after it has written them)
        early = "&" if register.startswith("v") else ""
        outputs.append(f'"={early}{{{register}}}"(accs[{t}])')
    outputs += ['[a_off] "+v"(a_offset)', '[b_off] "+v"(b_offset)', '[pairs] "+s"(step_pairs)']
    inputs = ['[ra0] "v"(read_a0)', '[ra1] "v"(read_a1)', '[rb0] "v"(read_b0)', '[rb1] "v"(read_b1)',
              '[rsrc_a] "s"(a_resource)', '[rsrc_b] "s"(b_resource)', '[a_step] "s"(a_row_step)',
              '[b_step] "s"(b_row_step)', '[fill0] "s"(fill_base)']
    if layout.nn:
        inputs += ['[fill0b] "s"(fill_base_b)', '[a_kstep] "s"(a_k_step)']
    clobbers = ['"memory"', '"scc"', f'"{SAVED_M0}"', f'"{OFFSET}"', f'"{FILL1}"', f'"{FILL1B}"']
    named = [n for n in range(layout.clobbered_v)
             if not layout.extra_acc_base <= n < layout.extra_acc_base + layout.extra_acc]
    clobbers += [f'"v{n}"' for n in named]
    if DROP & {"tovgpr", "dswrite", "staged"}:
        clobbers += [f'"v{n}"' for n in range(layout.clobbered_v, layout.clobbered_v + 4 * (layout.na + NB))]

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
    parser.add_argument("--drop", default="")
    parser.add_argument("--fill-every", type=int, default=FILL_EVERY)
    parser.add_argument("--order", default=ORDER)
    parser.add_argument("--reads", default=READS)
    arguments = parser.parse_args()
    DROP.update(item for item in arguments.drop.split(",") if item)
    globals()["FILL_EVERY"] = arguments.fill_every
    globals()["ORDER"] = arguments.order
    globals()["READS"] = arguments.reads
    experiments = DROP & {"tovgpr", "dswrite", "staged"}
    for na in (8, 10):
        if na == 10 and experiments:  # the register experiments need more registers than the 320-row tile leaves
            DROP.difference_update(experiments)
        layout = Layout(na)
        (arguments.out / f"wave4_loop_{layout.rows}x256.inc").write_text(statement(layout))
    if not experiments:
        (arguments.out / "wave4_loop_256x256_nn.inc").write_text(statement(Layout(8, nn=True)))


if __name__ == "__main__":
    main()
