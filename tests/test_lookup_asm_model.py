"""The generated phase body (tf-approximate_amd/csrc/gen_lookup_asm.py) waits for LDS and memory operations with
hand-counted s_waitcnt.  This test re-reads the emitted instruction text with an independent model of the hardware
counters (LDS operations and vector-memory loads each complete in issue order; s_waitcnt N lets the newest N stay
in flight; lgkmcnt is a 4-bit counter) and checks, on every control-flow path of every macro, that no instruction
touches a register an outstanding load has yet to write, that the counter never needs more than 15, and that
nothing is in flight when the macro ends."""
import importlib.util
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOKEN = re.compile(r"%\[\w+\]|v\[\d+:\d+\]|v\d+")


def _generator():
    path = os.path.join(ROOT, "tf-approximate_amd", "csrc", "gen_lookup_asm.py")
    spec = importlib.util.spec_from_file_location("gen_lookup_asm", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _instructions(macro_text):
    """The quoted assembly lines of the macro, in order: ("label", name) or ("ins", text)."""
    out = []
    for m in re.finditer(r'"([^"]*)\\n\\t"', macro_text):
        text = m.group(1).strip()
        if text.endswith(":"):
            out.append(("label", text[:-1]))
        else:
            out.append(("ins", text))
    return out


def _regs(token):
    if token.startswith("v["):
        a, b = token[2:-1].split(":")
        return ["v%d" % i for i in range(int(a), int(b) + 1)]
    return [token]


def _operands(text):
    regs = []
    for tok in TOKEN.findall(text):
        regs += _regs(tok)
    return regs


def _run(prog, nr):
    """The instructions a wavefront with `nr` pixels executes: the scalar compares against %[nr] are evaluated, the
    conditional branches follow them.  A branch on a condition code that something else has overwritten fails."""
    labels = {name: i for i, (kind, name) in enumerate(prog) if kind == "label"}
    pc, scc, trace = 0, None, []
    while pc < len(prog):
        kind, text = prog[pc]
        pc += 1
        if kind != "ins":
            continue
        op, args = text.split()[0], [a.strip() for a in text.split(None, 1)[1].split(",")] if " " in text else []
        if op == "s_branch":
            pc = labels[args[0]]
            continue
        if op.startswith("s_cbranch_scc"):
            assert scc is not None, "%r: the condition code is not that of a compare with %%[nr]" % text
            if scc == (op == "s_cbranch_scc1"):
                pc = labels[args[0]]
            continue
        if op.startswith("s_cmp"):
            value = [nr if a == "%[nr]" else int(a) for a in args]
            scc = {"s_cmp_eq_u32": value[0] == value[1], "s_cmp_lt_u32": value[0] < value[1]}[op]
        elif op.startswith("s_add") or op.startswith("s_sub") or op.startswith("s_and") or op.startswith("s_or"):
            scc = None
        trace.append(text)
    return trace


def _paths(prog, rows=None):
    """Every way through the macro: one per pixel count 0 .. rows."""
    if rows is None:
        rows = 1 + max(int(m.group(1)) for kind, text in prog if kind == "ins"
                       for m in [re.match(r"s_cmp_lt_u32 (\d+), %\[nr\]", text)] if m)
    return [_run(prog, nr) for nr in range(rows + 1)]


def _check_path(trace):
    lds, vm = [], []          # in-flight operations, oldest first: the set of registers each will write
    for text in trace:
        op = text.split()[0]
        if op == "s_waitcnt":
            for name, queue in (("lgkmcnt", lds), ("vmcnt", vm)):
                m = re.search(name + r"\((\d+)\)", text)
                if m:
                    del queue[:max(0, len(queue) - int(m.group(1)))]
            continue
        touched = _operands(text)
        pending = set().union(*lds, *vm) if (lds or vm) else set()
        clash = pending.intersection(touched)
        assert not clash, "%r touches %s while a load into it is in flight" % (text, sorted(clash))
        if op.startswith("ds_"):
            first = TOKEN.search(text).group(0)
            lds.append(set(_regs(first)) if op.startswith("ds_read") else set())
            assert len(lds) <= 15, "more than 15 LDS operations in flight at %r" % text
        elif op.startswith("buffer_load"):
            # a load with the lds modifier lands in LDS, not in a register (its only register is the address)
            vm.append(set() if text.rstrip().endswith(" lds") else set(_regs(TOKEN.search(text).group(0))))
    assert not lds and not vm, "operations still in flight at the end of the macro"


@pytest.mark.parametrize("nt", [16, 32, 64])
@pytest.mark.parametrize("buf", [0, 1])
def test_every_path_waits_for_what_it_uses(nt, buf):
    gen = _generator()
    prog = _instructions(gen.emit(nt, buf))
    assert sum(1 for kind, text in prog if kind == "ins" and text.startswith("ds_read_b128")) >= 8
    paths = _paths(prog)
    rows = 2 * (64 // nt)
    assert len(paths) == rows + 1        # 0 pixels, or the last pixel is pixel 0 .. rows-1
    for trace in paths:
        _check_path(trace)
    # a lane with r pixels issues 8 lookups per pixel
    counts = sorted(sum(1 for t in trace if t.startswith("ds_read_b128")) for trace in paths)
    assert counts == [8 * r for r in range(rows + 1)]


@pytest.mark.parametrize("buf", [0, 1])
def test_every_path_of_the_pre_expanded_phase_waits_for_what_it_uses(buf):
    """The phase that reads pre-expanded fills: 16 lookups per pixel (two activation dwords), eight loads that copy
    the next fill into LDS, two activation loads per pixel."""
    gen = _generator()
    prog = _instructions(gen.emit_px(buf))
    paths = _paths(prog)
    assert len(paths) == 9               # 0 pixels, or the last pixel is pixel 0 .. 7
    for nr, trace in enumerate(paths):
        _check_path(trace)
        assert sum(1 for t in trace if t.startswith("buffer_load_dwordx4") and t.endswith(" lds")) == 8
        # pixel 0's activations always (the kernel reads them when a tile starts), the others only where they exist
        loaded = sorted(TOKEN.search(t).group(0) for t in trace if t.startswith("buffer_load_dword "))
        assert loaded == sorted("%%[n%s%d]" % (k, r) for r in range(max(nr, 1)) for k in "fg")
        # the LDS destination register is written one instruction ahead of the load that uses it, at least
        for i, t in enumerate(trace):
            if t.startswith("buffer_load_dwordx4"):
                assert trace[i - 2].startswith("s_add_u32 m0,") and not trace[i - 1].startswith("s_add_u32 m0,")
    counts = sorted(sum(1 for t in trace if t.startswith("ds_read_b128")) for trace in paths)
    assert counts == [16 * r for r in range(9)]
    # buffer 1 is addressed through the instruction offset, buffer 0 without one; the fill lands in the other buffer
    reads = [t for t in max(paths, key=len) if t.startswith("ds_read_b128")]
    assert all(t.endswith("offset:65521") for t in reads) if buf else all("offset" not in t for t in reads)
    dests = sorted(int(t.split(",")[-1]) for t in max(paths, key=len) if t.startswith("s_add_u32 m0,"))
    assert dests == [(1 - buf) * 65536 + j * 1024 for j in range(8)]


def test_every_accumulator_gets_its_share_of_a_pre_expanded_fill():
    """A pre-expanded fill holds 8 input channels for each of 16 columns: every accumulator of every pixel receives
    eight entries, even columns from whole dwords, odd columns from high halves, and every landed dword is used once
    whole and once for its high half per unit (two units per pixel)."""
    gen = _generator()
    path = max(_paths(_instructions(gen.emit_px(0))), key=len)
    adds, uses = {}, {}
    for text in path:
        if text.startswith("v_add_u32_sdwa") or text.startswith("v_add3_u32"):
            toks = TOKEN.findall(text)
            dst, sources = toks[0], toks[2:]
            assert toks[1] == dst and dst.startswith("%[c")
            high = "WORD_1" in text
            adds.setdefault(dst, []).extend([high] * len(sources))
            for src in sources:
                uses.setdefault(src, []).append(high)
    assert len(adds) == 8 * 16
    for r in range(8):
        for j in range(16):
            kinds = adds["%%[c%d_%d]" % (r, j)]
            assert len(kinds) == 8 and all(k == bool(j & 1) for k in kinds)
    assert len(uses) == 32
    for src, kinds in uses.items():
        assert sorted(kinds) == [False] * 16 + [True] * 16, src


def test_the_model_notices_a_missing_wait():
    """The checker itself: dropping one s_waitcnt from a path must be reported."""
    gen = _generator()
    prog = _instructions(gen.emit(16, 0))
    path = max(_paths(prog), key=len)
    first_wait = next(i for i, t in enumerate(path) if t.startswith("s_waitcnt lgkmcnt"))
    broken = path[:first_wait] + path[first_wait + 1:]
    with pytest.raises(AssertionError):
        _check_path(broken)


@pytest.mark.parametrize("nt", [16, 32, 64])
def test_every_accumulator_gets_its_share_of_a_fill(nt):
    """A fill holds 64 / NT input channels for each of NT columns: on the path of a full lane every accumulator of
    every pixel must receive exactly that many table entries, half of the columns from the low halves of the dwords
    (add of whole dwords: one per v_add_u32, two per v_add3_u32) and half from the high halves (SDWA WORD_1), and
    every landed dword must be used exactly twice: once whole, once for its high half."""
    gen = _generator()
    rows = 2 * (64 // nt)
    path = max(_paths(_instructions(gen.emit(nt, 0))), key=len)
    adds, uses = {}, {}
    for text in path:
        if text.startswith("v_add_u32") or text.startswith("v_add3_u32"):
            toks = TOKEN.findall(text)
            dst = toks[0]
            if dst.startswith("%[c"):
                assert toks[1] == dst                       # accumulates in place
                sources = toks[2:]
                assert len(sources) == (2 if text.startswith("v_add3") else 1)
                high = "WORD_1" in text
                adds.setdefault(dst, []).extend([high] * len(sources))
                for src in sources:
                    uses.setdefault(src, []).append(high)
    assert len(adds) == rows * nt
    for r in range(rows):
        for j in range(nt):
            kinds = adds["%%[c%d_%d]" % (r, j)]
            assert len(kinds) == 64 // nt
            assert all(k == bool(j & 1) for k in kinds)
    # 32 landing registers, each read whole and for its high half once per pixel
    assert len(uses) == 32
    for src, kinds in uses.items():
        assert sorted(kinds) == [False] * rows + [True] * rows, src
    if nt < 64:    # three accumulate operations per four entries
        n_ops = sum(1 for t in path if t.startswith("v_add_u32") or t.startswith("v_add3_u32"))
        n_acc = sum(1 for t in path if (t.startswith("v_add_u32") or t.startswith("v_add3_u32")) and "%[c" in t)
        assert n_acc == rows * 64 * 3 // 4 and n_ops >= n_acc


# ---- the phase of the kernel without a barrier between fills -------------------------------------------------------

PENDING, ISSUED, COUNTED = 1000, 0xfffffffe, 0xffffffff


def _run_free(prog, nr, tgt0, fire=-1, land=0):
    """One way through PHASE_PXF for a wavefront with `nr` pixels.  tgt0 is the state of the fill the phase starts
    with: PENDING (a count the other buffer's events have yet to reach: the poll number `fire` is the first that sees
    it there, -1 = none does), ISSUED or COUNTED.  The `land`-th look at the vector-memory counter after the issue is
    the first that finds no load in flight.  Returns the trace, the number of polls consumed and the final state."""
    labels = {name: i for i, (kind, name) in enumerate(prog) if kind == "label"}
    pc, scc, trace, polls, tgt, looks = 0, None, [], 0, tgt0, 0
    while pc < len(prog):
        kind, text = prog[pc]
        pc += 1
        if kind != "ins":
            continue
        op = text.split()[0]
        args = [a.strip() for a in text.split(None, 1)[1].split(",")] if " " in text else []
        if op == "s_branch":
            pc = labels[args[0]]
            continue
        if op.startswith("s_cbranch_scc"):
            assert scc is not None, "%r: the condition code is stale" % text
            if scc == (op == "s_cbranch_scc1"):
                pc = labels[args[0]]
            continue
        if op == "s_cmp_ge_u32" and args[0] == "%[tgt]":
            polls += 1
            scc = tgt != PENDING and tgt >= int(args[1], 16)
        elif op == "s_cmp_ge_u32":
            assert args == ["%[seen]", "%[tgt]"] and tgt == PENDING
            scc = 0 <= fire <= polls - 1
        elif op == "s_cmp_eq_u32" and args[0] == "%[tgt]":
            assert args[1] == "-1"
            scc = tgt == COUNTED
        elif op.startswith("s_cmp"):
            value = [nr if a == "%[nr]" else int(a) for a in args]
            scc = {"s_cmp_eq_u32": value[0] == value[1], "s_cmp_lt_u32": value[0] < value[1]}[op]
        elif op == "s_and_b32":
            assert trace[-1].startswith("s_getreg_b32 %[stmp], hwreg(HW_REG_IB_STS)") and args[:2] == ["%[stmp]"] * 2
            assert int(args[2], 16) == 0x00c0000f        # the six bits of the vector-memory counter in IB_STS
            scc = looks < land                           # non-zero: loads in flight
            looks += 1
        elif op.startswith("s_add") or op.startswith("s_sub") or op.startswith("s_or"):
            scc = None
        elif op == "s_mov_b32" and args[0] == "%[tgt]":
            tgt = int(args[1], 16) & 0xffffffff
        trace.append(text)
    return trace, polls, tgt


def _free_cases():
    for nr in range(9):
        for fire in range(-1, 9):
            for land in range(4):
                yield nr, PENDING, fire, land
        for land in range(10):
            yield nr, ISSUED, -1, land
        yield nr, COUNTED, -1, 0


def test_every_path_of_the_phase_without_barriers_waits_for_what_it_uses():
    gen = _generator()
    prog = _instructions(gen.emit_pxf())
    assert prog[0] == ("ins", "s_mov_b32 %[seen], 0")
    n = 0
    for nr, tgt0, fire, land in _free_cases():
        trace, polls, tgt = _run_free(prog, nr, tgt0, fire, land)
        _check_path(trace)
        # one poll per pixel: the 4-byte read of the other buffer's events and the look at what it returned
        assert polls == nr and sum(1 for t in trace if t.startswith("ds_read_b32")) == nr
        assert sum(1 for t in trace if t.startswith("ds_read_b128")) == 16 * nr
        loads = sum(1 for t in trace if t.startswith("buffer_load_dwordx4") and t.endswith(" lds"))
        counts = sum(1 for t in trace if t.startswith("ds_add_u32"))
        if tgt0 == PENDING:
            issued = 0 <= fire < nr
            counted = issued and fire + 1 + land < nr       # the looks start with the poll after the issue
        else:
            issued, counted = True, tgt0 == ISSUED and land < nr
        assert loads == (8 if issued and tgt0 == PENDING else 0), (nr, tgt0, fire, loads)
        assert counts == (1 if counted else 0), (nr, tgt0, fire, land, counts)
        assert tgt == (COUNTED if counted or tgt0 == COUNTED else ISSUED if issued else PENDING)
        for i, t in enumerate(trace):
            if t.startswith("buffer_load_dwordx4"):
                # the LDS destination register is written one instruction ahead of the load that uses it, at least
                assert trace[i - 2].startswith("s_add_u32 m0,") and not trace[i - 1].startswith("s_add_u32 m0,")
            if t.startswith("ds_add_u32"):
                # a single lane adds, and the wavefront has all its lanes back right after
                assert trace[i - 2:i] == ["s_mov_b64 %[sx], exec", "s_mov_b64 exec, 1"]
                assert trace[i + 1] == "s_mov_b64 exec, %[sx]"
        assert sum(1 for t in trace if " exec" in t) == 3 * counts
        dests = sorted(int(t.split(",")[-1]) for t in trace if t.startswith("s_add_u32 m0, %[edst],"))
        assert dests == ([j * 1024 for j in range(8)] if loads else [])
        loaded = sorted(TOKEN.search(t).group(0) for t in trace if t.startswith("buffer_load_dword "))
        assert loaded == sorted("%%[n%s%d]" % (k, r) for r in range(max(nr, 1)) for k in "fg")
        n += 1
    assert n == 9 * (10 * 4 + 10 + 1)


def test_the_phase_without_barriers_looks_up_and_accumulates_every_entry_once():
    """Data flow of the longest path, symbolically.  A lookup is (activation register, chunk register, selector): the
    row comes from byte `step` of the pixel's FIRST or SECOND dword, the 16-byte chunk from the chunk register of the
    same half.  The dword d of step s holds columns (s % 2) * 8 + 2 d (low half) and + 1 (high half); each accumulator
    must receive the eight entries of its column (four steps of each half) and nothing else, which also shows that no
    landing register is overwritten before its adds and no address register between its v_perm_b32 and its read."""
    gen = _generator()
    trace, _, _ = _run_free(_instructions(gen.emit_pxf()), 8, COUNTED)
    value, acc = {}, {}
    for text in trace:
        op, toks = text.split()[0], TOKEN.findall(text)
        if op == "v_perm_b32":
            m = re.fullmatch(r"v_perm_b32 (v\d+), %\[([fg])(\d)\], %\[ch(\d)([abc])\], %\[s(\d)\]", text)
            assert m, text
            dst, half, r, chalf, third, step = m.group(1), "fg".index(m.group(2)), int(m.group(3)), int(m.group(4)), \
                m.group(5), int(m.group(6))
            assert chalf == half and third == "abc"[step // 3]
            value[dst] = ("address", r, half, step)
        elif op == "ds_read_b128":
            kind, r, half, step = value[toks[1]]
            assert kind == "address" and "offset" not in text
            for d, reg in enumerate(_regs(toks[0])):
                value[reg] = ("entry", r, half, step, d)
        elif op in ("v_add3_u32", "v_add_u32_sdwa"):
            dst, sources = toks[0], toks[2:]
            assert toks[1] == dst and dst.startswith("%[c")
            for src in sources:
                assert value[src][0] == "entry", text
                acc.setdefault(dst, []).append(value[src][1:] + ("WORD_1" in text,))
        elif op in ("v_mov_b32", "v_add_u32", "ds_read_b32", "buffer_load_dword"):
            value[toks[0]] = ("other",)
        else:
            assert not op.startswith("v_") or op == "v_readfirstlane_b32", text
    assert len(acc) == 8 * 16
    for r in range(8):
        for j in range(16):
            want = sorted((r, half, step, (j % 8) // 2, bool(j & 1))
                          for half in range(2) for step in range(j // 8, 8, 2))
            assert sorted(acc["%%[c%d_%d]" % (r, j)]) == want, (r, j)
