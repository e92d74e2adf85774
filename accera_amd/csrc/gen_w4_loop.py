#!/usr/bin/env python3
"""Writes gemm_mfma16w4_loop.inc: the K loop of the four-wave 256x256 GEMM kernel as one block of
gfx950 assembly per layout of matrix B.

    python3 gen_w4_loop.py > gemm_mfma16w4_loop.inc

One wave per SIMD owns a 128x128 piece of the output tile: 8 x 8 blocks of 16x16, 256 accumulator
registers, which only fit when they live in a[0:255] for the whole loop while v[128:255] hold
two sets of operand fragments.  The compiler's register allocator does not keep that split on
its own (it moves accumulators between the two files and spills), so the loop is laid out by
hand: registers are fixed, and each k-step of 64 bytes is

    s_waitcnt lgkmcnt(4)            fragments of this step are in registers (all but A's last four)
    32 MFMAs (rows 0..63 of the wave tile, column by column with the rows back and forth, so that
    consecutive MFMAs share one operand: 0.6-1 % faster than row by row), the 8 fill instructions of the step three ahead
    and their address arithmetic spread between them, at most two per MFMA
    s_waitcnt vmcnt(2 tiles' fills); s_barrier  the tile of the next step has landed for every wave
    32 MFMAs (rows 64..127), the fragment reads of the next step between them, one per MFMA

The four LDS stages rotate with the k-step, so the body is written out for four steps; the last
four steps (no more fills, then no more reads) are a second copy.  A number of k-steps that is not
a multiple of four enters the body in the middle (see loop()); at least four steps.

Register use (besides the operands the C++ side passes in):
    a[0:255]    accumulators, block (i, j) at a[(i*TN+j)*4 .. +3] (TN = 8 blocks of columns per wave, 6 for the 192-wide tile)
    v[128:191]  fragments of even steps: B blocks 0..7 (v128..), A blocks 0..7 (v160..)
    v[192:255]  fragments of odd steps
    v[104:121]  LDS read addresses of the upper two stages (the 16-bit offset field reaches 64 KB)
    v[114:127], v103  column-major A only: the read addresses of A's blocks 1..7 (lower two stages) and 0..7 (upper two)
    s[72:73], s[74:75]  fill pointers of A and B (the next tile to fetch); s[76:77], s[80:81] scratch pointers; s78 loop count;
    s79 row offset while C is loaded
"""
B_TILE = 16384     # B's tile follows A's (256 rows x 64 bytes) inside a stage
FRAG = 1024        # 16 rows x 64 bytes (K-contiguous operand)
TN = 8             # blocks of 16 columns per wave: 8 (256-wide tile) or 6 (192-wide, K-contiguous B only)
STAGE = 32768      # A's tile + B's tile (2 * TN * 16 rows x 64 bytes)
RELAX_STORES = 47  # stores per thread the relaxed first k-steps of a later tile count on (see loop(): 2 tiles' fills + 47 = 63)
A_LAYOUT = "kc"    # "kc": A row-major (K contiguous); "mc16" / "mc8": A as it lies in memory when column-major (M contiguous)
A_LOW = ["%[a_rd]", "v122", "v123", "v124", "v125", "v126", "v127", "v103"]  # column-major A: read addresses of the lower two stages


def set_width(tn):
    global TN, STAGE
    TN = tn
    STAGE = B_TILE + 2 * tn * FRAG


def acc(i, j):
    n = (i * TN + j) * 4
    return f"a[{n}:{n + 3}]"


def bfrag(buf, j):
    n = 128 + buf * 64 + j * 4
    return n


def afrag(buf, i):
    n = 160 + buf * 64 + i * 4
    return n


def mfma(i, j, buf):
    b, a = bfrag(buf, j), afrag(buf, i)
    return f'MFMA " {acc(i, j)}, v[{b}:{b + 3}], v[{a}:{a + 3}], {acc(i, j)}\\n"'


def line(s):
    return f'"{s}\\n"'


def read_a(x, stage, buf):
    n = afrag(buf, x)
    if A_LAYOUT == "kc":
        base = "%[a_rd]" if stage < 2 else "v104"
        off = (stage & 1) * STAGE + x * FRAG
        return [line(f"ds_read_b128 v[{n}:{n + 3}], {base} offset:{off}")]
    # column-major A is staged as it lies in memory (M contiguous) and read like a row-major B
    op = "ds_read_b64_tr_b16" if A_LAYOUT == "mc16" else "ds_read_b64_tr_b8"
    base = A_LOW[x] if stage < 2 else f"v{114 + x}"
    out = []
    for q in range(2):
        off = (stage & 1) * STAGE + q * 2048
        out.append(line(f"{op} v[{n + 2 * q}:{n + 2 * q + 1}], {base} offset:{off}"))
    return out


def read_b(x, stage, buf, b_layout):
    n = bfrag(buf, x)
    if b_layout in ("kc", "kcp"):
        base = "%[b_rd0]" if stage < 2 else "v105"
        off = (stage & 1) * STAGE + B_TILE + x * FRAG
        return [line(f"ds_read_b128 v[{n}:{n + 3}], {base} offset:{off}")]
    # B as it lies in memory (N contiguous): two transposing reads per block, 4 (16-bit) or 8 (8-bit)
    # k rows = 2048 bytes apart; every block has its own address (the swizzle is an XOR)
    op = "ds_read_b64_tr_b16" if b_layout == "mc16" else "ds_read_b64_tr_b8"
    base = f"%[b_rd{x}]" if stage < 2 else f"v{106 + x}"
    out = []
    for q in range(2):
        off = (stage & 1) * STAGE + B_TILE + q * 2048
        out.append(line(f"{op} v[{n + 2 * q}:{n + 2 * q + 1}], {base} offset:{off}"))
    return out


def fill(f, stage, b_layout):
    """Fill instruction f (0..3 A, 4.. B) of a K tile as a list of MFMA slots: pointer, M0, the load (the MFMA
    between the M0 write and the load is the wait state M0 needs; the last pass also advances the pointer)."""
    if f < 4:
        ptr, d, s, tile, g, last = "s[72:73]", "%[da]", "%[sa]", 0, f, 3
        lane = "%[a_off]" if (A_LAYOUT == "kc" or g % 2 == 0) else "%[a_off1]"
    else:
        g = f - 4
        ptr, d, s, tile, last = "s[74:75]", "%[db]", "%[sb]", B_TILE, (2 * TN * FRAG) // 4096 - 1
        lane = "%[b_off0]" if (b_layout in ("kc", "kcp") or g % 2 == 0) else "%[b_off1]"
    slots = []
    if g == 0:
        slots.append([line(f"s_mov_b64 s[76:77], {ptr}")])
    else:
        slots.append([line(f"s_add_u32 s76, s76, {d}"), line("s_addc_u32 s77, s77, 0")])
    slots.append([line(f"s_add_u32 m0, %[ldsb], {stage * STAGE + tile + g * 4096}")])
    slots.append([line(f"global_load_lds_dwordx4 {lane}, s[76:77]")])
    if g == last:  # advance to the next K tile
        lo, hi = (72, 73) if f < 4 else (74, 75)
        slots[-1] += [line(f"s_add_u32 s{lo}, s{lo}, {s}"), line(f"s_addc_u32 s{hi}, s{hi}, 0")]
    return slots


def kc_fills(pos, half):
    """Fill instructions of one k-step of the "kcp" scheme (B K-contiguous, fills paired), as lists per MFMA slot.  Both operands' K tiles are
    half cache lines, so both are fetched as pairs of neighbouring requests: A's tile t+3 last in odd steps and first
    in even ones (as for the other layouts), and B two tiles at a time, t+2 and t+3 pass by pass, on even steps only."""
    nb = (2 * TN * FRAG) // 4096
    slots = []
    for g in range(4):  # A, tile t+3 -> stage (pos+3) % 4
        first = [line("s_mov_b64 s[76:77], s[72:73]")] if g == 0 else [line("s_add_u32 s76, s76, %[da]"), line("s_addc_u32 s77, s77, 0")]
        slots.append(first + [line(f"s_add_u32 m0, %[ldsb], {((pos + 3) % 4) * STAGE + g * 4096}")])
        slots.append([line("global_load_lds_dwordx4 %[a_off], s[76:77]")])
    slots[-1] += [line("s_add_u32 s72, s72, %[sa]"), line("s_addc_u32 s73, s73, 0")]
    if pos % 2:
        return [[] for _ in range(half - len(slots))] + slots
    for g in range(nb):  # B, tiles t+2 and t+3 -> stages (pos+2) % 4 and (pos+3) % 4
        if g == 0:
            ptrs = [line("s_mov_b64 s[76:77], s[74:75]"), line("s_add_u32 s80, s74, %[sb]"), line("s_addc_u32 s81, s75, 0")]
        else:
            ptrs = [line("s_add_u32 s76, s76, %[db]"), line("s_addc_u32 s77, s77, 0"), line("s_add_u32 s80, s80, %[db]"), line("s_addc_u32 s81, s81, 0")]
        slots.append(ptrs + [line(f"s_add_u32 m0, %[ldsb], {((pos + 2) % 4) * STAGE + B_TILE + g * 4096}")])
        slots.append([line("global_load_lds_dwordx4 %[b_off0], s[76:77]"),
                      line(f"s_add_u32 m0, %[ldsb], {((pos + 3) % 4) * STAGE + B_TILE + g * 4096}")])
        slots.append([line("global_load_lds_dwordx4 %[b_off0], s[80:81]")])
    slots[-1] += [line("s_add_u32 s74, s74, %[sb]"), line("s_addc_u32 s75, s75, 0"), line("s_add_u32 s74, s74, %[sb]"), line("s_addc_u32 s75, s75, 0")]
    assert len(slots) <= half
    return slots + [[] for _ in range(half - len(slots))]


def kc_wait(pos, tiles_left):
    """vmcnt before the barrier of a k-step with K-contiguous B: how many fills issued after the next tile's last one
    may still be in flight.  tiles_left: K tiles after this step's (>= 3 inside the body)."""
    nb = (2 * TN * FRAG) // 4096
    if tiles_left >= 3:
        return 8 + 2 * nb if pos % 2 == 0 else 5   # even: A(t+2), A(t+3), B(t+2), B(t+3); odd: B(t+2)'s last pass, A(t+3)
    assert pos == 4 - 1 - tiles_left                 # the closing steps sit at positions 1 and 2
    return 1 if tiles_left == 2 else 0              # position 1: B's last tile's last pass; position 2: nothing


def step(pos, do_fill, wait, last, b_layout):
    buf, nxt, fst = pos % 2, (pos + 1) % 4, (pos + 3) % 4
    # fragments of B and of A's first four blocks are in registers (the last four reads may still be in flight)
    out = [line("s_waitcnt lgkmcnt(4)")]
    # (columns back and forth: consecutive MFMAs always share one operand)
    order = []
    for h in range(2):  # rows 0..3 of blocks before the barrier, 4..7 after; inside a half column by column, rows back and forth
        for j in range(TN):
            rows = range(4 * h, 4 * h + 4)
            order += [(i, j) for i in (rows if j % 2 == 0 else reversed(rows))]
    half = 4 * TN
    extra = [[] for _ in range(half)]
    if do_fill and b_layout == "kcp":
        extra = kc_fills(pos, half)
    elif do_fill:
        # A's fills come last in odd steps and first in even ones: the two 64-byte halves of a 128-byte
        # line of a K-contiguous operand belong to k-steps 2m and 2m+1, filled in steps 2m-3 and 2m-2;
        # requested back to back, the second half is still in the CU's vector cache
        nb = (2 * TN * FRAG) // 4096
        fills = list(range(4 + nb)) if pos % 2 == 0 else list(range(4, 4 + nb)) + list(range(4))
        # fill() chains the scratch pointer from one pass of an operand to its next: passes must come in order
        assert [f for f in fills if f < 4] == [0, 1, 2, 3] and [f for f in fills if f >= 4] == list(range(4, 4 + nb))
        per = half // len(fills)  # MFMA slots per fill: 4 (256-wide) or 3 (192-wide)
        for n, f in enumerate(fills):
            for k, ins in enumerate(fill(f, fst, b_layout)):
                extra[n * per + k] += ins
    for s, (i, j) in enumerate(order[:half]):
        out.append(mfma(i, j, buf))
        out += extra[s]
    out.append(line("s_waitcnt lgkmcnt(0)"))
    if not last:
        out.append(line(f"s_waitcnt vmcnt({wait})"))
        out.append(line("s_barrier"))
    reads = []
    if not last:
        for x in range(TN):
            reads += read_b(x, nxt, buf ^ 1, b_layout)
        for x in range(8):
            reads += read_a(x, nxt, buf ^ 1)
    for s, (i, j) in enumerate(order[half:]):
        out.append(mfma(i, j, buf))
        if s < len(reads):
            out.append(reads[s])
    return out


def loop(b_layout, persist=False):
    """persist: the loop of a workgroup that walks several output tiles.  Two bits of %[flags]:
    bit 0  the closing steps go on fetching: the first three K tiles of the workgroup's NEXT output tile (from
           %[pa_n] / %[pb_n]) go into the stages the closing steps leave behind, so that the workgroup finds them in LDS
           (or on the way) after its write-back.  Only for an entry at position 0 (a number of k-steps that is a
           multiple of four: tile s of the next output tile then belongs in stage s), not for the paired-fill scheme.
    bit 1  the stores of the previous tile's write-back (at least RELAX_STORES per thread) were issued after the fills
           of this tile's K tiles 1 and 2 and may still be in flight: the first four k-steps are a copy of the body
           whose first two waits allow for them (memory operations complete in the order issued, so a wait count
           that does not know of the stores would wait for nearly all of them).  Entry at position 0 and at least one
           trip through the body (the copy counts as one)."""
    assert not (persist and b_layout == "kcp")
    out = [line("s_mov_b64 s[72:73], %[pa]"), line("s_mov_b64 s[74:75], %[pb]"), line("s_mov_b32 s78, %[groups]")]
    if A_LAYOUT == "kc":
        out.append(line(f"v_add_u32 v104, {2 * STAGE}, %[a_rd]"))
    else:
        # block x of the wave's rows lies x * 32 (16-bit) or x * 16 (8-bit) bytes further along every k row of the tile, and
        # the swizzle is an XOR on those address bits (rows of the tile start on multiples of their length)
        assert TN == 8
        for x in range(1, 8):
            out.append(line(f"v_xor_b32 {A_LOW[x]}, {x * (32 if A_LAYOUT == 'mc16' else 16)}, %[a_rd]"))
        for x in range(8):
            out.append(line(f"v_add_u32 v{114 + x}, {2 * STAGE}, {A_LOW[x]}"))
    if b_layout in ("kc", "kcp"):
        out.append(line(f"v_add_u32 v105, {2 * STAGE}, %[b_rd0]"))
    else:
        for x in range(8):
            out.append(line(f"v_add_u32 v{106 + x}, {2 * STAGE}, %[b_rd{x}]"))
    # accumulators: zero, or (C += A*B with 32-bit C) the tile of C, loaded straight into the AGPR file
    # (or nothing: a 16-bit C has been widened into them by the code before the loop)
    out += [line("s_cmp_eq_u32 %[accum], 0"), line("s_cbranch_scc1 3f"), line("s_cmp_eq_u32 %[accum], 2"), line("s_cbranch_scc1 4f"),
            line("s_mov_b32 s79, 0")]
    for i in range(8):
        for j in range(TN):
            n = (i * TN + j) * 4
            out.append(line(f"buffer_load_dwordx4 a[{n}:{n + 3}], %[c_off], %[c_rsrc], s79 offen offset:{j * 64}"))
        out.append(line("s_add_u32 s79, s79, %[c_row16]"))
    out += [line("s_waitcnt vmcnt(0)"), line("s_branch 4f"), line("3:")]
    for n in range(32 * TN):
        out.append(line(f"v_accvgpr_write_b32 a{n}, 0"))
    out.append(line("4:"))
    # Entry.  The last k-step always runs at position 3 of the closing copy, so the first one starts at position
    # p0 = (4 - steps % 4) % 4: its tile lies in LDS stage p0 (the code before the loop put it there), its fragments
    # go to register set p0 % 2, and the body is entered at that position (labels 5, 6, 7 = positions 1, 2, 3).
    def first_reads(pos):
        r = []
        for x in range(TN):
            r += read_b(x, pos, pos % 2, b_layout)
        for x in range(8):
            r += read_a(x, pos, pos % 2)
        return r + [line("s_nop 7")]
    out += [line("s_cmp_eq_u32 %[p0], 0"), line("s_cbranch_scc1 10f"), line("s_cmp_eq_u32 %[p0], 1"), line("s_cbranch_scc1 11f"),
            line("s_cmp_eq_u32 %[p0], 2"), line("s_cbranch_scc1 12f")]
    out += first_reads(3) + [line("s_branch 7f"), line("11:")]
    out += first_reads(1) + [line("s_branch 5f"), line("12:")]
    out += first_reads(2) + [line("s_branch 6f"), line("10:")]
    out += first_reads(0)
    per_tile = 4 + (2 * TN * FRAG) // 4096  # fill instructions per K tile and thread
    kc = b_layout == "kcp"
    if persist:
        # in flight, oldest first, at the wait of step 0: tile 1, tile 2, the stores, tile 3; at that of step 1: tile 2, the
        # stores, tiles 3 and 4; from step 2 on the tile waited for is younger than the stores
        relaxed = min(63, 2 * per_tile + RELAX_STORES)
        out += [line("s_bitcmp1_b32 %[flags], 1"), line("s_cbranch_scc0 13f")]
        out += step(0, True, relaxed, False, b_layout) + step(1, True, relaxed, False, b_layout)
        out += step(2, True, 2 * per_tile, False, b_layout) + step(3, True, 2 * per_tile, False, b_layout)
        out += [line("s_sub_u32 s78, s78, 1"), line("13:")]
    out += [line("s_cmp_eq_u32 s78, 0"), line("s_cbranch_scc1 2f"), line("1:")]
    for pos in range(4):
        if pos:
            out.append(line(f"{4 + pos}:"))
        out += step(pos, True, kc_wait(pos, 3) if kc else 2 * per_tile, False, b_layout)
    out += [line("s_sub_u32 s78, s78, 1"), line("s_cmp_lg_u32 s78, 0"), line("s_cbranch_scc1 1b"), line("2:")]
    out += step(0, True, kc_wait(0, 3) if kc else 2 * per_tile, False, b_layout)
    if persist:
        # closing steps that go on fetching: the fill pointers move to the next output tile; waits as in the body
        out += [line("s_bitcmp1_b32 %[flags], 0"), line("s_cbranch_scc0 8f"),
                line("s_mov_b64 s[72:73], %[pa_n]"), line("s_mov_b64 s[74:75], %[pb_n]")]
        out += step(1, True, 2 * per_tile, False, b_layout)
        out += step(2, True, 2 * per_tile, False, b_layout)
        out += step(3, True, 0, True, b_layout)
        out += [line("s_branch 9f"), line("8:")]
    out += step(1, False, kc_wait(1, 2) if kc else per_tile, False, b_layout)
    out += step(2, False, 0, False, b_layout)
    out += step(3, False, 0, True, b_layout)
    if persist:
        out.append(line("9:"))
    out += [line("s_nop 15"), line("s_nop 15")]
    return out


def main():
    print("// Generated by gen_w4_loop.py; do not edit.  The K loop of gemm_mfma16w4_kernel, one macro per")
    print("// layout of B (K contiguous, plain or with paired fills / N contiguous 16-bit / N contiguous 8-bit); MFMA is the mnemonic.")
    # kcp: K-contiguous B with its half-line fills paired (two K tiles per even step); measured ahead of the plain
    # scheme for the 192-wide tile and for int8, behind it for 16-bit inputs on the 256-wide tile
    for name, tn in (("kc", 8), ("kcp", 8), ("mc16", 8), ("mc8", 8), ("kcp", 6)):
        set_width(tn)
        body = loop(name)
        print(f"#define ACC950_W4_LOOP_{name.upper()}{'' if tn == 8 else tn}(MFMA) \\")
        print(" \\\n".join("    " + s for s in body))
        print()
    # the same loops for a workgroup that walks several output tiles (closing steps that prefetch the next tile)
    for name in ("kc", "mc16", "mc8"):
        set_width(8)
        body = loop(name, persist=True)
        print(f"#define ACC950_W4_LOOP_{name.upper()}_P(MFMA) \\")
        print(" \\\n".join("    " + s for s in body))
        print()
    main_a_mc()


def main_a_mc():
    """The loops for a column-major A (one macro per pair of layouts), for one tile per workgroup and for a workgroup that
    walks several tiles (_P: closing steps that prefetch the next tile)."""
    global A_LAYOUT
    for persist in (False, True):
        for a_name, b_name in (("mc16", "kc"), ("mc16", "mc16"), ("mc8", "kc"), ("mc8", "mc8")):
            set_width(8)
            A_LAYOUT = a_name
            body = loop(b_name, persist=persist)
            A_LAYOUT = "kc"
            print(f"#define ACC950_W4_LOOP_{b_name.upper()}_A{a_name.upper()}{'_P' if persist else ''}(MFMA) \\")
            print(" \\\n".join("    " + s for s in body))
            print()


if __name__ == "__main__":
    main()
