"""The K loop of the four-wave GEMM kernel is generated assembly text (accera_amd/csrc/gen_w4_loop.py ->
gemm_mfma16w4_loop.inc).  These checks read that text on the CPU: the include in the tree is what the
generator writes, and every k-step keeps the invariants the kernel's correctness (and the safety of its
global addresses) rests on -- one MFMA per accumulator block, fragment reads that land in the other
register set and stay inside the LDS stage they are meant for, fill passes of an operand in order (the
scratch pointer is chained from pass to pass), one pointer advance per operand and step, and wait
counts that match the number of fills in flight."""
import importlib.util
import os
import re

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "accera_amd", "csrc")


def _gen():
    spec = importlib.util.spec_from_file_location("gen_w4_loop", os.path.join(CSRC, "gen_w4_loop.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _text(lines):
    """Generator lines -> plain instructions ('MFMA a[..], ..' for the MFMA macro lines)."""
    out = []
    for l in lines:
        m = re.match(r'^MFMA " (.*)\\n"$', l)
        out.append("MFMA " + m.group(1) if m else re.match(r'^"(.*)\\n"$', l).group(1))
    return out


def test_include_in_the_tree_is_what_the_generator_writes(capsys):
    g = _gen()
    g.main()
    assert capsys.readouterr().out == open(os.path.join(CSRC, "gemm_mfma16w4_loop.inc")).read()


@pytest.mark.parametrize("layout,tn", [("kc", 8), ("kcp", 8), ("mc16", 8), ("mc8", 8), ("kcp", 6)])
def test_every_k_step_keeps_its_invariants(layout, tn):
    g = _gen()
    g.set_width(tn)
    stage_bytes, b_tile = g.STAGE, g.B_TILE
    assert stage_bytes == 16384 + tn * 2048 and 4 * stage_bytes <= 160 * 1024
    nb = tn * 2048 // 4096                      # fill passes of B per K tile
    per_tile = 4 + nb
    for pos in range(4):
        for do_fill, wait, last in ((True, g.kc_wait(pos, 3) if layout == "kcp" else 2 * per_tile, False), (False, per_tile, False),
                                    (False, 0, False), (False, 0, True)):
            ins = _text(g.step(pos, do_fill, wait, last, layout))
            buf, nxt, fst = pos % 2, (pos + 1) % 4, (pos + 3) % 4
            # ---- MFMAs: every accumulator block once, operands from this step's register set
            blocks = []
            for i in ins:
                m = re.match(r"MFMA a\[(\d+):(\d+)\], v\[(\d+):(\d+)\], v\[(\d+):(\d+)\], a\[(\d+):(\d+)\]$", i)
                if not m:
                    continue
                d0, d1, b0, b1, a0, a1, c0, c1 = map(int, m.groups())
                assert (d0, d1) == (c0, c1) and d1 == d0 + 3 and d0 % 4 == 0 and d1 < 32 * tn
                blk = d0 // 4
                bi, bj = divmod(blk, tn)
                assert b0 == 128 + buf * 64 + bj * 4 and b1 == b0 + 3      # B's fragment: first operand
                assert a0 == 160 + buf * 64 + bi * 4 and a1 == a0 + 3      # A's fragment: second operand
                blocks.append(blk)
            assert sorted(blocks) == list(range(8 * tn))
            # ---- fragment reads of the next step: other register set, inside the next step's LDS stage
            reads = [i for i in ins if i.startswith("ds_read")]
            assert len(reads) == (0 if last else 8 + (tn if layout in ("kc", "kcp") else 2 * tn))
            written = set()
            for r in reads:
                m = re.match(r"(ds_read_b128|ds_read_b64_tr_b16|ds_read_b64_tr_b8) v\[(\d+):(\d+)\], (\S+) offset:(\d+)$", r)
                op, v0, v1, base, off = m.group(1), int(m.group(2)), int(m.group(3)), m.group(4), int(m.group(5))
                assert 128 + (buf ^ 1) * 64 <= v0 and v1 < 128 + (buf ^ 1) * 64 + 64, "reads must not touch the registers in use"
                assert not written & set(range(v0, v1 + 1))
                written |= set(range(v0, v1 + 1))
                upper = not base.startswith("%")                  # v104.. hold the addresses of stages 2 and 3
                assert upper == (nxt >= 2)
                assert off < 65536                                # the instruction's offset field
                in_stage = off - (nxt & 1) * stage_bytes
                assert 0 <= in_stage < stage_bytes
                is_b = 128 + (buf ^ 1) * 64 <= v0 < 160 + (buf ^ 1) * 64
                assert (in_stage >= b_tile) == is_b
                assert (op == "ds_read_b128") == (layout in ("kc", "kcp") or not is_b)
            assert len(written) == (0 if last else (8 + tn) * 4)
            # ---- fills of the tile three steps ahead
            loads = [n for n, i in enumerate(ins) if i.startswith("global_load_lds")]
            for n in loads:
                assert ins[n - 1].startswith("MFMA"), "one instruction between the M0 write and its use"
                assert any(i.startswith("s_add_u32 m0,") for i in ins[max(0, n - 8):n - 1])
            if layout == "kcp":
                # (K-contiguous B with paired fills: A's tile t+3 every step, B's tiles t+2 and t+3 on even positions; addresses, stages and
                # waits of this scheme are checked over whole loops by the model below)
                assert len(loads) == ((4 + (2 * nb if pos % 2 == 0 else 0)) if do_fill else 0)
                if do_fill:
                    assert max(loads) < ins.index("s_barrier")
            else:
                assert len(loads) == (per_tile if do_fill else 0)
            if do_fill and layout != "kcp":
                first_mfma_after_barrier = ins.index("s_barrier")
                assert max(loads) < first_mfma_after_barrier      # all issued before this step's wait
                seen = {"a": [], "b": []}
                chain = None                                       # operand the scratch pointer currently belongs to
                m0 = None
                advanced = []
                for n, i in enumerate(ins[:first_mfma_after_barrier]):
                    if i.startswith("s_mov_b64 s[76:77], "):
                        chain = {"s[72:73]": "a", "s[74:75]": "b"}[i.split(", ")[1]]
                        assert not seen[chain], "an operand's first pass starts from its tile pointer"
                    elif i.startswith("s_add_u32 s76, s76, "):
                        assert chain == {"%[da]": "a", "%[db]": "b"}[i.split(", ")[2]] and seen[chain]
                        assert ins[n + 1] == "s_addc_u32 s77, s77, 0"
                    elif i.startswith("s_add_u32 m0, %[ldsb], "):
                        m0 = int(i.split(", ")[2])
                    elif i.startswith("global_load_lds"):
                        assert ins[n - 1].startswith("MFMA"), "one instruction between the M0 write and its use"
                        lane = i.split()[1].rstrip(",")
                        g_pass = len(seen[chain])
                        tile = 0 if chain == "a" else b_tile
                        assert m0 == fst * stage_bytes + tile + g_pass * 4096
                        assert m0 + 4096 <= 4 * stage_bytes
                        if chain == "a":
                            assert lane == "%[a_off]"
                        else:
                            assert lane == ("%[b_off0]" if layout == "kc" or g_pass % 2 == 0 else "%[b_off1]")
                        seen[chain].append(g_pass)
                        m0 = None
                    elif re.match(r"s_add_u32 s7[24], s7[24], %\[s[ab]\]$", i):
                        op = "a" if "s72" in i else "b"
                        assert i.endswith("%[sa]") == (op == "a")
                        assert len(seen[op]) == (4 if op == "a" else nb), "the tile pointer moves on after the operand's last pass"
                        advanced.append(op)
                assert seen == {"a": [0, 1, 2, 3], "b": list(range(nb))} and sorted(advanced) == ["a", "b"]
            # ---- waits
            assert ins[0] == "s_waitcnt lgkmcnt(4)"
            assert ("s_barrier" in ins) == (not last)
            if not last:
                b = ins.index("s_barrier")
                assert ins[b - 1] == f"s_waitcnt vmcnt({wait})" and ins[b - 2] == "s_waitcnt lgkmcnt(0)"


@pytest.mark.parametrize("layout,tn", [("kc", 8), ("kcp", 8), ("mc16", 8), ("kcp", 6)])
def test_whole_loop_shape(layout, tn):
    """Preamble, four-step body with its back branch, and the four closing steps (one with fills, three without)."""
    g = _gen()
    g.set_width(tn)
    ins = _text(g.loop(layout))
    per_tile = 4 + tn * 2048 // 4096
    assert ins.count("1:") == 1 and ins.count("2:") == 1 and ins.index("1:") < ins.index("s_cbranch_scc1 1b") < ins.index("2:")
    # the body can be entered at each of its four positions (a step count that is not a multiple of four); every entry
    # first reads the fragments of the first tile from the stage of that position into that position's register set
    assert ins.index("1:") < ins.index("5:") < ins.index("6:") < ins.index("7:") < ins.index("s_cbranch_scc1 1b")
    entry = ins[ins.index("4:"):ins.index("1:")]
    for label, jump, pos in ((None, "s_branch 7f", 3), ("11:", "s_branch 5f", 1), ("12:", "s_branch 6f", 2), ("10:", "s_cbranch_scc1 2f", 0)):
        start = entry.index(label) + 1 if label else entry.index("s_cbranch_scc1 12f") + 1
        block = entry[start:entry.index(jump, start)]
        reads = [i for i in block if i.startswith("ds_read")]
        assert len(reads) == 8 + (tn if layout in ("kc", "kcp") else 2 * tn)
        for r in reads:
            m = re.match(r"\S+ v\[(\d+):(\d+)\], (\S+) offset:(\d+)$", r)
            v0, base, off = int(m.group(1)), m.group(3), int(m.group(4))
            assert 128 + (pos % 2) * 64 <= v0 < 192 + (pos % 2) * 64
            assert (not base.startswith("%")) == (pos >= 2) and 0 <= off - (pos & 1) * g.STAGE < g.STAGE
    step_starts = [ins.index("1:"), ins.index("5:"), ins.index("6:"), ins.index("7:")]
    assert all(ins[n + 1] == "s_waitcnt lgkmcnt(4)" for n in step_starts)
    body = [i for i in ins[ins.index("1:"):ins.index("2:")] if i not in ("5:", "6:", "7:")]
    tail = ins[ins.index("2:"):]
    assert sum(i.startswith("MFMA") for i in body) == 4 * 8 * tn == sum(i.startswith("MFMA") for i in tail)
    assert body.count("s_barrier") == 4 and tail.count("s_barrier") == 3
    assert sum(i.startswith("global_load_lds") for i in body) == 4 * per_tile
    nb = tn * 2048 // 4096
    if layout == "kcp":  # the closing copy's first step fetches A's last tile and B's last two
        assert sum(i.startswith("global_load_lds") for i in tail) == 4 + 2 * nb
        assert [i for i in tail if i.startswith("s_waitcnt vmcnt")] == [f"s_waitcnt vmcnt({8 + 2 * nb})", "s_waitcnt vmcnt(1)", "s_waitcnt vmcnt(0)"]
    else:
        assert sum(i.startswith("global_load_lds") for i in tail) == per_tile
        assert [i for i in tail if i.startswith("s_waitcnt vmcnt")] == [f"s_waitcnt vmcnt({2 * per_tile})", f"s_waitcnt vmcnt({per_tile})", "s_waitcnt vmcnt(0)"]
    # accumulators: zeroed, or loaded from C block by block (64 bytes per block and row group, 16 rows further per row of blocks)
    pre = ins[:ins.index("1:")]
    assert sum(i.startswith("v_accvgpr_write_b32") for i in pre) == 32 * tn
    c_loads = [i for i in pre if i.startswith("buffer_load_dwordx4")]
    assert len(c_loads) == 8 * tn
    for n, i in enumerate(c_loads):
        m = re.match(r"buffer_load_dwordx4 a\[(\d+):(\d+)\], %\[c_off\], %\[c_rsrc\], s79 offen offset:(\d+)$", i)
        assert int(m.group(1)) == n * 4 and int(m.group(2)) == n * 4 + 3 and int(m.group(3)) == (n % tn) * 64
    assert pre.count("s_add_u32 s79, s79, %[c_row16]") == 8
    # the loop ends with enough idle cycles for the last MFMA results to be readable
    assert ins[-2:] == ["s_nop 15", "s_nop 15"]


def _run_fills(g, layout, tn, KT, b_tiles_before_loop, persist=False, flags=0, stores_in_flight=0):
    """Executes the scalar side of the loop text for KT k-steps: follows the branches, keeps the fill pointers as
    numbers and records every global_load_lds as (operand, K tile, pass, LDS stage).  The code before the loop
    has issued A's tiles 0..2 and B's tiles 0..b_tiles_before_loop-1; pa / pb point at the next tiles."""
    g.set_width(tn)
    ins = _text(g.loop(layout, persist) if persist else g.loop(layout))
    DA, DB, SA, SB = 1 << 20, 1 << 21, 1 << 30, 1 << 34      # distinct powers of two: an address decodes uniquely
    NEXT = 1 << 49                                            # marks the panels of the workgroup's next output tile
    p0 = (4 - KT % 4) % 4
    groups = KT // 4 - 1 + (1 if KT % 4 else 0)
    env = {"%[pa]": 3 * SA, "%[pb]": (1 << 50) + b_tiles_before_loop * SB, "%[groups]": groups, "%[p0]": p0, "%[accum]": 0,
           "%[da]": DA, "%[db]": DB, "%[sa]": SA, "%[sb]": SB, "%[ldsb]": 0, "%[c_row16]": 0,
           "%[pa_n]": NEXT, "%[pb_n]": (1 << 50) + NEXT, "%[flags]": flags}
    labels = {}
    for n, i in enumerate(ins):
        if re.match(r"^\d+:$", i):
            labels.setdefault(i[:-1], []).append(n)
    reg, scc, m0, pc, fills, steps = {}, 0, None, 0, [], 0
    nb_ = tn * 2048 // 4096
    # fills in flight, oldest first: what the code before the loop issued (tile by tile, A's passes then B's), then the loop's
    issued = []
    for t in range(3):
        issued += [("a", t, p) for p in range(4)]
        if t < b_tiles_before_loop:
            issued += [("b", t, p) for p in range(nb_)]
    if b_tiles_before_loop > 3:
        issued += [("b", t, p) for t in range(3, b_tiles_before_loop) for p in range(nb_)]
    # stores of the previous output tile's write-back, issued after these fills (a workgroup that walks several tiles)
    issued += [("store", n, 0) for n in range(stores_in_flight)]

    def val(tok):
        tok = tok.strip()
        if tok in env:
            return env[tok]
        if re.match(r"^s\d+$", tok):
            return reg.get(tok, 0)
        return int(tok, 0)

    def pair(tok):  # s[a:b] or an operand
        m = re.match(r"s\[(\d+):(\d+)\]", tok.strip())
        return (reg.get("s" + m.group(1), 0) | (reg.get("s" + m.group(2), 0) << 32)) if m else env[tok.strip()]

    while pc < len(ins):
        i = ins[pc]
        pc += 1
        op, _, rest = i.partition(" ")
        a = [x.strip() for x in rest.split(",")] if rest else []
        if op == "s_mov_b64":
            m = re.match(r"s\[(\d+):(\d+)\]", a[0])
            v = pair(rest.split(",", 1)[1])
            reg["s" + m.group(1)], reg["s" + m.group(2)] = v & 0xffffffff, v >> 32
        elif op == "s_mov_b32":
            reg[a[0]] = val(a[1])
        elif op == "s_add_u32":
            t = val(a[1]) + val(a[2])
            scc = t >> 32
            if a[0] == "m0":
                m0 = t & 0xffffffff
            else:
                reg[a[0]] = t & 0xffffffff
        elif op == "s_addc_u32":
            t = val(a[1]) + val(a[2]) + scc
            scc, reg[a[0]] = t >> 32, t & 0xffffffff
        elif op == "s_sub_u32":
            reg[a[0]] = val(a[1]) - val(a[2])
        elif op == "s_cmp_eq_u32":
            scc = int(val(a[0]) == val(a[1]))
        elif op == "s_cmp_lg_u32":
            scc = int(val(a[0]) != val(a[1]))
        elif op == "s_bitcmp1_b32":
            scc = (val(a[0]) >> val(a[1])) & 1
        elif op in ("s_cbranch_scc1", "s_cbranch_scc0", "s_branch"):
            if op == "s_branch" or scc == (op == "s_cbranch_scc1"):
                lab, way = a[0][:-1], a[0][-1]
                cands = labels[lab]
                pc = min(c for c in cands if c >= pc) if way == "f" else max(c for c in cands if c < pc)
        elif op == "global_load_lds_dwordx4":
            addr = pair(rest.split(",", 1)[1])
            operand = "b" if addr >> 50 else "a"       # (bit 50 marks B's address space in this model)
            addr &= (1 << 50) - 1
            ahead = bool(addr & NEXT)                  # a fetch for the next output tile
            addr &= NEXT - 1
            stride, delta = (SB, DB) if operand == "b" else (SA, DA)
            tile, within = divmod(addr, stride)
            if ahead:
                tile += KT                             # K tile s of the next output tile is numbered KT + s
            assert within % delta == 0
            stage, in_stage = divmod(m0, g.STAGE)
            assert in_stage == (g.B_TILE if operand == "b" else 0) + (within // delta) * 4096
            fills.append((operand, tile, within // delta, stage))
            issued.append((operand, tile, within // delta))
            m0 = None
        elif op == "s_waitcnt" and a and a[0].startswith("vmcnt(") and steps:
            # loads complete in order: all but the youngest N are done.  The tile of the next k-step must be among them.
            n_out = int(a[0][6:-1])
            done = set(issued[:len(issued) - n_out]) if n_out else set(issued)
            nxt_tile = steps                                   # this is k-step steps-1; the barrier that follows publishes the next tile
            if nxt_tile < KT:
                need = {("a", nxt_tile, p) for p in range(4)} | {("b", nxt_tile, p) for p in range(nb_)}
                assert need <= done, (steps - 1, sorted(need - done))
        elif op == "s_waitcnt" and a and a[0].startswith("lgkmcnt(4)"):
            steps += 1
    return fills, steps, p0


@pytest.mark.parametrize("layout,tn", [("kc", 8), ("kcp", 8), ("mc16", 8), ("kcp", 6)])
@pytest.mark.parametrize("KT", [4, 5, 6, 7, 8, 9, 10, 11, 12, 23, 128])
def test_fill_addresses_over_a_whole_k_loop(layout, tn, KT):
    """Every pass of every K tile from 3 on is filled exactly once, from the address of that tile and pass, into
    the LDS stage its k-step will read ((tile + entry position) mod 4), and nothing beyond the last tile is touched."""
    g = _gen()
    p0 = (4 - KT % 4) % 4
    # with paired fills a K-contiguous B is fetched two tiles at a time on the even positions of the body: the code before the loop issues
    # B's tiles 0 and 1, and tile 2 as well when the first k-step sits at an odd position
    b_before = 3 if layout != "kcp" else 2 + (p0 & 1)
    fills, steps, p0 = _run_fills(g, layout, tn, KT, b_before)
    nb = tn * 2048 // 4096
    assert steps == KT
    want = sorted([("a", t, p, (t + p0) % 4) for t in range(3, KT) for p in range(4)] +
                  [("b", t, p, (t + p0) % 4) for t in range(b_before, KT) for p in range(nb)])
    assert sorted(fills) == want


@pytest.mark.parametrize("layout", ["kc", "mc16", "mc8"])
@pytest.mark.parametrize("KT", [4, 8, 12, 128])
@pytest.mark.parametrize("flags,stores", [(0, 0), (1, 0), (2, 64), (3, 64), (3, 47), (2, 500)])
def test_loop_of_a_workgroup_that_walks_several_tiles(layout, KT, flags, stores):
    """The loops with closing steps that fetch ahead (entry at position 0 only).  Bit 0 of the flags: the three
    closing steps fill K tiles 0..2 of the next output tile into stages 0..2, nothing else changes.  Bit 1: the first four
    k-steps are the copy whose waits allow for the previous tile's stores; the model keeps those stores in flight
    between the fills of K tile 2 and those of K tile 3 and still finds every k-step's tile landed at its barrier
    (memory operations complete in the order issued)."""
    g = _gen()
    if flags & 2 and KT < 8:
        pytest.skip("the relaxed copy of the first four k-steps counts as one trip through the body: at least eight k-steps")
    fills, steps, p0 = _run_fills(g, layout, 8, KT, 3, persist=True, flags=flags, stores_in_flight=stores)
    assert steps == KT and p0 == 0
    last = KT + 3 if flags & 1 else KT
    want = sorted([(o, t, p, t % 4) for o in "ab" for t in range(3, last) for p in range(4)])
    assert sorted(fills) == want
    # the closing steps that fetch ahead are the body's steps: same text up to the waits and the missing last barrier
    ins = _text(g.loop(layout, persist=True))
    assert ins.count("s_bitcmp1_b32 %[flags], 0") == 1 and ins.count("s_bitcmp1_b32 %[flags], 1") == 1
    assert sum(i.startswith("MFMA") for i in ins) == 64 * (4 + 4 + 1 + 3 + 3)   # relaxed copy, body, closing step 0, the two sets of closing steps
    relaxed = [i for i in ins[ins.index("s_bitcmp1_b32 %[flags], 1"):ins.index("13:")] if i.startswith("s_waitcnt vmcnt")]
    assert relaxed == ["s_waitcnt vmcnt(63)", "s_waitcnt vmcnt(63)", "s_waitcnt vmcnt(16)", "s_waitcnt vmcnt(16)"]
    assert g.RELAX_STORES + 16 == 63


def test_relaxed_first_steps_need_the_stores_they_count_on():
    """The model notices a wait that is too loose: with fewer stores in flight than the relaxed copy counts on, the
    tile of the second k-step is not known to have landed."""
    g = _gen()
    with pytest.raises(AssertionError):
        _run_fills(g, "mc8", 8, 8, 3, persist=True, flags=2, stores_in_flight=40)


@pytest.mark.parametrize("a_layout,b_layout", [("mc16", "kc"), ("mc16", "mc16"), ("mc8", "kc"), ("mc8", "mc8")])
def test_loops_for_a_column_major_a(a_layout, b_layout):
    """A staged as it lies in memory (M contiguous): its fragments come from transposing reads, two per block, from
    per-block addresses the preamble derives from block 0's; its fill passes alternate between two lane offsets."""
    g = _gen()
    g.set_width(8)
    g.A_LAYOUT = a_layout
    try:
        ins = _text(g.loop(b_layout))
        steps = {pos: _text(g.step(pos, True, 16, False, b_layout)) for pos in range(4)}
    finally:
        g.A_LAYOUT = "kc"
    # ---- preamble: blocks 1..7 of the lower stages by XOR, all eight of the upper stages 2 * STAGE further
    pre = ins[:ins.index("4:")]
    unit = 32 if a_layout == "mc16" else 16
    low = ["%[a_rd]"] + [None] * 7
    for i in pre:
        m = re.match(r"v_xor_b32 (v\d+), (\d+), %\[a_rd\]$", i)
        if m:
            x = int(m.group(2)) // unit
            assert int(m.group(2)) == x * unit and 1 <= x <= 7 and low[x] is None
            low[x] = m.group(1)
    assert None not in low and len(set(low)) == 8
    up = {}
    for i in pre:
        m = re.match(rf"v_add_u32 (v\d+), {2 * g.STAGE}, (\S+)$", i)
        if m and m.group(2) in low:
            up[low.index(m.group(2))] = m.group(1)
    assert sorted(up) == list(range(8))
    regs = [int(r[1:]) for r in low[1:] + list(up.values())]
    b_regs = set(range(106, 114)) if b_layout != "kc" else {105}
    assert len(set(regs)) == 15 and all(100 <= r < 128 for r in regs) and not set(regs) & b_regs, "registers the loop owns, none shared with B's"
    assert not any("v104" in i for i in ins)
    # ---- every step: 16 reads of A into the other register set, inside A's tile of the next stage
    op = "ds_read_b64_tr_b16" if a_layout == "mc16" else "ds_read_b64_tr_b8"
    for pos, st in steps.items():
        buf, nxt = pos % 2, (pos + 1) % 4
        assert st[0] == "s_waitcnt lgkmcnt(4)"
        reads = [i for i in st if i.startswith("ds_read")]
        assert len(reads) == 16 + (8 if b_layout == "kc" else 16) and len(reads) <= 32
        assert all(st[n - 1].startswith("MFMA") for n, i in enumerate(st) if i.startswith("ds_read")), "one read per MFMA slot"
        a_reads = []
        for r in reads:
            m = re.match(r"(\S+) v\[(\d+):(\d+)\], (\S+) offset:(\d+)$", r)
            v0 = int(m.group(2))
            if v0 >= 160 + (buf ^ 1) * 64 and v0 < 192 + (buf ^ 1) * 64:
                a_reads.append((m.group(1), v0, int(m.group(3)), m.group(4), int(m.group(5))))
        assert len(a_reads) == 16 and reads[-4:] == [r for r in reads if any(f"v[{a[1]}:" in r for a in a_reads[-4:])], "A's last reads close the step"
        for n, (o, v0, v1, base, off) in enumerate(a_reads):
            x, q = divmod(n, 2)
            assert o == op and v0 == 160 + (buf ^ 1) * 64 + x * 4 + 2 * q and v1 == v0 + 1
            assert base == (low[x] if nxt < 2 else up[x])
            assert off == (nxt & 1) * g.STAGE + q * 2048 and off + 2048 <= (nxt & 1) * g.STAGE + g.B_TILE
        # fills of A: passes 0..3 in order, even passes with one lane offset, odd ones with the other
        lanes = [i.split()[1].rstrip(",") for i in st if i.startswith("global_load_lds") and "a_off" in i]
        assert lanes == ["%[a_off]", "%[a_off1]", "%[a_off]", "%[a_off1]"]


@pytest.mark.parametrize("a_layout,b_layout", [("mc16", "kc"), ("mc16", "mc16"), ("mc8", "kc"), ("mc8", "mc8")])
@pytest.mark.parametrize("KT,flags,stores", [(8, 0, 0), (12, 1, 0), (128, 3, 64), (8, 2, 64), (12, 3, 47), (128, 2, 500)])
def test_column_major_a_loops_of_a_workgroup_that_walks_several_tiles(a_layout, b_layout, KT, flags, stores):
    """The same loops for a workgroup that walks several output tiles: closing steps that fetch the next tile's K tiles
    0..2, first k-steps whose waits allow for the previous tile's stores -- the scalar side behaves as for a row-major A,
    and the text around it is the one-tile loop's (same preamble of per-block read addresses, same reads per step)."""
    g = _gen()
    g.A_LAYOUT = a_layout
    try:
        fills, steps, p0 = _run_fills(g, b_layout, 8, KT, 3, persist=True, flags=flags, stores_in_flight=stores)
        walk, one = _text(g.loop(b_layout, persist=True)), _text(g.loop(b_layout))
    finally:
        g.A_LAYOUT = "kc"
    assert steps == KT and p0 == 0
    last = KT + 3 if flags & 1 else KT
    assert sorted(fills) == sorted([(o, t, p, t % 4) for o in "ab" for t in range(3, last) for p in range(4)])
    assert walk[:walk.index("4:")] == one[:one.index("4:")], "same preamble: read addresses, accumulators"
    assert sum(i.startswith("MFMA") for i in walk) == 64 * (4 + 4 + 1 + 3 + 3)
    op = "ds_read_b64_tr_b16" if a_layout == "mc16" else "ds_read_b64_tr_b8"
    per_step = 16 + (8 if b_layout == "kc" else 16)
    # every k-step but the last of either set of closing steps reads the next step's fragments: 4 + 4 + 1 + 2 + 2 steps
    assert sum(i.startswith("ds_read") for i in walk[walk.index("10:"):]) == per_step * (1 + 4 + 4 + 1 + 2 + 2)
    assert sum(i.startswith(op) for i in walk[walk.index("13:"):]) >= 16 * 9


def test_block_addresses_of_a_column_major_tile_differ_by_an_xor():
    """What the preamble above relies on: with the tile's k rows starting on multiples of their length, the LDS address
    of block x's transposing read is block 0's with x * 32 (16-bit) or x * 16 (8-bit) XORed in, for every lane."""
    for es, row_bytes in ((2, 512), (1, 256)):
        cpr = row_bytes // 16
        def swizzle(row, c):
            if es == 2:
                return c ^ ((((row & 3) << 2) | (((row >> 3) & 1) << 1)) & (cpr - 1))
            return c ^ ((((row & 7) << 1) | ((row >> 4) & 1)) & (cpr - 1))
        for base in (0, 1024, 32768, 5 * 16384):      # start of the tile in LDS
            for wr0 in (0, 128):
                for lane in range(64):
                    kg, li = lane >> 4, lane & 15
                    def addr(x):
                        if es == 2:
                            col_byte, k = (wr0 + x * 16 + (li & 3) * 4) * 2, kg * 8 + (li >> 2)
                        else:
                            col_byte, k = wr0 + x * 16 + (li & 1) * 8, kg * 16 + (li >> 1)
                        return base + k * row_bytes + swizzle(k, col_byte >> 4) * 16 + (col_byte & 15)
                    for x in range(8):
                        assert addr(x) == addr(0) ^ (x * 16 * es)
