#!/usr/bin/env python3
"""Generates lookup_asm.inc: the inline-assembly body of one phase of the dense LUT-GEMM kernel.

    python gen_lookup_asm.py > lookup_asm.inc

For each tile width NT (16, 32, 64 columns) and each parity BUF of the phase it emits one macro
PHASE_NT<NT>_B<BUF>(...) that a wavefront executes once per fill p (BUF = p & 1), between two workgroup
barriers.  The macro interleaves, in one instruction stream with hand-counted s_waitcnt:

  lookups   all lookups of fill p for the first NR (wave-uniform, 0..R) output pixels of the lane, out of
            expanded-row buffer BUF.  A pixel needs eight 16-byte reads of the expanded row of its activation
            code.  The LDS address of step s is ONE v_perm_b32 (byte 1 <- activation code: the rows of the two
            buffers interleave, 256 bytes apart; byte 0 <- the lane's chunk offset).  The reads run through a
            rolling window of eight that does not drain between pixels.  Each arrived chunk is accumulated
            with eight VALU adds, one per table entry: the entry in the high half of a dword through the SDWA
            source selector, the one in the low half by adding the whole dword (the surplus, 65536 times the
            high entries, is subtracted once behind the last phase).  Step s accumulates into column group
            s % (NT / 8).
  loads     table rows of fill p+2 -> staged-row buffer BUF, straight from memory into LDS (buffer loads with the
            lds modifier: M0 carries the LDS address of the wavefront's 1 KiB, every lane adds its 16 bytes;
            addresses from CODES), filter codes of fill p+3 -> CODES, activations of fill p+1 -> ANEXT; all waited
            for at the end of the macro.
  derive    the staged rows of fill p+1 (buffer BUF^1) are transposed into expanded-row buffer BUF^1: two
            items per lane, each four 8-byte reads, eight v_perm_b32 and four 8-byte writes.
            Loads and derive are cut into micro-operations and one of them is slotted in behind every
            16-byte chunk of the lookups (loads first, so that their latency runs under the lookups), so that
            the memory pipeline and the LDS see them spread out instead of as one burst per wavefront right
            after the barrier; what a wavefront with few pixels has not placed by its last chunk follows
            behind it.

NT = 16: a fill holds 4 input channels and the activation dword is used as it is.
NT = 32 / 64: a fill holds 2 / 1 channels; the dword is first rotated right by SHIFT bits (an SGPR) so that
         the channels of this fill are its low bytes.

LDS instructions complete in order, so "wait until operation X has completed" is s_waitcnt lgkmcnt(number
of LDS operations issued after X); the generator keeps the issue queue and derives every count from it.
The landing registers and temporaries are fixed VGPRs declared as clobbers, because inline-asm operands
cannot name the dwords of a register tuple.
"""

DERIVE_IN = 204            # 8 registers: four 8-byte staged-row reads of one derive item
DERIVE_OUT = 212           # 6 registers: transposed dwords (two more reuse DERIVE_IN)
ROT_TEMP = 218             # rotated activation dword of the pixel whose reads are being issued
WR_TEMP = 219              # expanded-row write address of a derive item
ADDR_BASE = 220            # 4 rolling address temporaries: v220..v223
TEMP_BASE = 224            # 8 x 4 landing registers: v224..v255
CLOBBER_FIRST = DERIVE_IN


class Stream:
    """Instruction list plus the queue of LDS operations in flight."""

    def __init__(self, lines=None, fifo=None, seq=0):
        self.lines = lines if lines is not None else []
        self.fifo = list(fifo) if fifo is not None else []
        self.seq = seq

    def fork(self):
        return Stream(self.lines, self.fifo, self.seq + 100000)

    def ins(self, text):
        self.lines.append('"%s\\n\\t"' % text)

    def label(self, text):
        self.lines.append('"%s:\\n\\t"' % text)

    def lds(self, text):
        if len(self.fifo) == 15:     # lgkmcnt is a 4-bit counter: retire the oldest operation first
            self.wait(self.fifo[0])
        self.ins(text)
        self.seq += 1
        self.fifo.append(self.seq)
        return self.seq

    def wait(self, op):
        """Wait until LDS operation `op` (and everything older) has completed."""
        if op not in self.fifo:
            return
        i = self.fifo.index(op)
        self.ins("s_waitcnt lgkmcnt(%d)" % (len(self.fifo) - 1 - i))
        del self.fifo[:i + 1]

    def drain(self):
        self.ins("s_waitcnt vmcnt(0) lgkmcnt(0)")
        self.fifo = []


def emit(nt, buf):
    sets = nt // 8
    rows = 2 * (64 // nt)
    other = buf ^ 1

    def rotate(st, r):
        if nt == 16:
            return "%%[a%d]" % r
        st.ins("v_alignbit_b32 v%d, %%[a%d], %%[a%d], %%[shift]" % (ROT_TEMP, r, r))
        return "v%d" % ROT_TEMP

    def read(st, src, step):
        b = TEMP_BASE + 4 * step
        va = ADDR_BASE + (step % 4)
        st.ins("v_perm_b32 v%d, %s, %%[%s], %%[s%d]" % (va, src, "cha" if step < 4 else "chb", step))
        off = " offset:128" if buf else ""
        return st.lds("ds_read_b128 v[%d:%d], v%d%s" % (b, b + 3, va, off))

    def adds(st, r, steps):
        """Accumulates the chunks of `steps` (one step, or two steps with the same column group)."""
        g = steps[0] % sets
        for d in range(4):
            even = "%%[c%d_%d]" % (r, g * 8 + 2 * d)
            odd = "%%[c%d_%d]" % (r, g * 8 + 2 * d + 1)
            regs = [TEMP_BASE + 4 * step + d for step in steps]
            # the whole dwords: the accumulator of the even column collects lo + 65536 * hi (mod 2^32); the kernel
            # takes 65536 * (sum of hi) off again behind the last phase
            if len(regs) == 2:
                st.ins("v_add3_u32 %s, %s, v%d, v%d" % (even, even, regs[0], regs[1]))
            else:
                st.ins("v_add_u32 %s, %s, v%d" % (even, even, regs[0]))
            for reg in regs:
                st.ins("v_add_u32_sdwa %s, %s, v%d dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1"
                       % (odd, odd, reg))

    # steps of a pixel that are accumulated together, in consumption order
    if sets == 8:
        groups = [(s,) for s in range(8)]
    else:
        groups = [(s, s + sets) for base in range(0, 8, 2 * sets) for s in range(base, base + sets)]

    def prime(st):
        src = rotate(st, 0)
        return [read(st, src, s) for s in range(8)]

    def body(st, r, pending, with_next, state):
        """Accumulate pixel r (its reads are `pending`); with_next: refill the window with pixel r + 1.
        One auxiliary micro-operation is slotted in behind every chunk."""
        nxt = [None] * 8
        src = rotate(st, r + 1) if with_next else None
        for steps in groups:
            # LDS operations complete in order: waiting for the youngest read of the group covers the others
            st.wait(max((pending[s] for s in steps), key=lambda op: st.fifo.index(op) if op in st.fifo else -1))
            adds(st, r, steps)
            for s in steps:
                if with_next:
                    nxt[s] = read(st, src, s)
                aux_step(st, state)
        return nxt

    # ---- auxiliary work, cut into micro-operations that are spread over the chunk slots ----
    def row_load(j):         # staged rows [buf] of fill p+2 <- table[code][16 bytes of this lane], memory -> LDS
        def f(st, state):
            t = ADDR_BASE + 3    # the lookup address of a step is consumed by the read right behind it
            st.ins("s_add_u32 m0, %%[stm], %d" % (j * 8192 + buf * 32768))
            st.ins("v_lshlrev_b32 v%d, 9, %%[k%d]" % (t, j))
            st.ins("v_and_or_b32 v%d, v%d, %%[cmask], %%[sto]" % (t, t))
            st.ins("buffer_load_dwordx4 v%d, %%[tab], 0 offen lds" % t)
            st.ins("s_nop 0")
        return f

    def code_load(j):        # filter codes of fill p+3
        return lambda st, state: st.ins("buffer_load_ushort %%[k%d], %%[cvo], %%[wq], %%[cso] offen offset:%d" % (j, 32 * j))

    def act_load(r):         # activations of fill p+1
        return lambda st, state: st.ins("buffer_load_dword %%[n%d], %%[t%d], %%[xq], %%[qoff] offen" % (r, r))

    def derive_reads(item):
        def f(st, state):
            o = 64 * other  # staged-row buffer [other], in units of 512 bytes
            st.lds("ds_read2st64_b64 v[%d:%d], %%[rd%d] offset0:%d offset1:%d"
                   % (DERIVE_IN, DERIVE_IN + 3, item, o, o + 1))
            state["dr"] = st.lds("ds_read2st64_b64 v[%d:%d], %%[rd%d] offset0:%d offset1:%d"
                                 % (DERIVE_IN + 4, DERIVE_IN + 7, item, o + 2, o + 3))
        return f

    def derive_consume(item):
        def f(st, state):
            i, o = DERIVE_IN, DERIVE_OUT
            st.wait(state["dr"])
            # in: v[i:i+1] slot 0, v[i+2:i+3] slot 1, v[i+4:i+5] slot 2, v[i+6:i+7] slot 3 (two codes per dword)
            st.ins("v_perm_b32 v%d, v%d, v%d, %%[plo]" % (o + 0, i + 2, i + 0))
            st.ins("v_perm_b32 v%d, v%d, v%d, %%[plo]" % (o + 1, i + 6, i + 4))
            st.ins("v_perm_b32 v%d, v%d, v%d, %%[phi]" % (o + 2, i + 2, i + 0))
            st.ins("v_perm_b32 v%d, v%d, v%d, %%[phi]" % (o + 3, i + 6, i + 4))
            st.ins("v_perm_b32 v%d, v%d, v%d, %%[plo]" % (o + 4, i + 3, i + 1))
            st.ins("v_perm_b32 v%d, v%d, v%d, %%[plo]" % (o + 5, i + 7, i + 5))
            st.ins("v_perm_b32 v%d, v%d, v%d, %%[phi]" % (i + 0, i + 3, i + 1))
            st.ins("v_perm_b32 v%d, v%d, v%d, %%[phi]" % (i + 1, i + 7, i + 5))
            if other:
                st.ins("v_add_u32 v%d, 128, %%[wr%d]" % (WR_TEMP, item))
                wa = "v%d" % WR_TEMP
            else:
                wa = "%%[wr%d]" % item
            st.lds("ds_write2st64_b64 %s, v[%d:%d], v[%d:%d] offset0:0 offset1:32" % (wa, o, o + 1, o + 2, o + 3))
            st.lds("ds_write2st64_b64 %s, v[%d:%d], v[%d:%d] offset0:64 offset1:96" % (wa, o + 4, o + 5, i, i + 1))
        return f

    def both(f, g):
        return lambda st, state: (f(st, state), g(st, state))

    # Global loads first: a wavefront with few pixels has few chunk slots, and what does not fit behind a chunk is
    # issued behind the last one, right in front of the wait for it.  Then the expansion of fill p+1, the reads of
    # a derive item eight slots ahead of its transposes.
    aux = []
    for j in range(4):
        aux += [row_load(j)]
    aux += [both(code_load(0), code_load(1)), both(code_load(2), code_load(3))]   # code_load j overwrites what row_load j read
    aux += [both(act_load(r), act_load(r + 1)) for r in range(0, rows, 2)]
    aux += [derive_reads(0)]
    for _ in range(7):
        aux.append(lambda st, state: None)
    aux += [both(derive_consume(0), derive_reads(1))]
    for _ in range(7):
        aux.append(lambda st, state: None)
    aux += [derive_consume(1)]

    def aux_step(st, state):
        if state["pos"] < len(aux):
            aux[state["pos"]](st, state)
            state["pos"] += 1

    def aux_rest(st, state):
        while state["pos"] < len(aux):
            aux_step(st, state)

    main = Stream()
    main.ins("s_cmp_eq_u32 %[nr], 0")
    main.ins("s_cbranch_scc1 Lzero_%=")
    pending = prime(main)
    state = {"pos": 0, "dr": None}
    forks = []
    for r in range(rows):
        if r < rows - 1:
            main.ins("s_cmp_lt_u32 %d, %%[nr]" % (r + 1))
            main.ins("s_cbranch_scc0 Llast%d_%%=" % r)
            forks.append((r, main.fork(), list(pending), dict(state)))
            pending = body(main, r, pending, True, state)
        else:
            body(main, r, pending, False, state)
    aux_rest(main, state)
    main.drain()
    main.ins("s_branch Lend_%=")
    for r, st, pend, stt in forks:
        st.label("Llast%d_%%=" % r)
        body(st, r, pend, False, stt)
        aux_rest(st, stt)
        st.drain()
        st.ins("s_branch Lend_%=")
    zero = Stream(main.lines)
    zero.label("Lzero_%=")
    aux_rest(zero, {"pos": 0, "dr": None})
    zero.drain()
    zero.label("Lend_%=")

    outs = ['[c%d_%d] "+v"(ACC[%d][%d])' % (r, i, r, i) for r in range(rows) for i in range(nt)]
    outs += ['[k%d] "+v"(CODES[%d])' % (j, j) for j in range(4)]
    outs += ['[n%d] "=&v"(ANEXT[%d])' % (r, r) for r in range(rows)]
    inp = ['[a%d] "v"(ACUR[%d])' % (r, r) for r in range(rows)]
    inp += ['[t%d] "v"(TAPOFF[%d])' % (r, r) for r in range(rows)]
    inp += ['[s%d] "v"(SEL[%d])' % (i, i) for i in range(8)]
    inp += ['[cha] "v"(CHA)', '[chb] "v"(CHB)', '[nr] "s"(NR)']
    inp += ['[stm] "s"(STM)', '[sto] "v"(STO)', '[cvo] "v"(CVO)']
    inp += ['[rd0] "v"(RD[0])', '[rd1] "v"(RD[1])', '[wr0] "v"(WR[0])', '[wr1] "v"(WR[1])']
    inp += ['[plo] "s"(0x05040100u)', '[phi] "s"(0x07060302u)', '[cmask] "s"(0x01fffe00u)']
    inp += ['[tab] "s"(TAB)', '[wq] "s"(WQ)', '[xq] "s"(XQ)', '[cso] "s"(CSO)', '[qoff] "s"(QOFF)']
    if nt != 16:
        inp.append('[shift] "s"(SHIFT)')
    clob = ", ".join('"v%d"' % r for r in range(CLOBBER_FIRST, TEMP_BASE + 32))
    body_text = " \\\n        ".join(main.lines)
    args = "ACC, ACUR, ANEXT, TAPOFF, CODES, SEL, CHA, CHB, NR, SHIFT, STM, STO, CVO, RD, WR, TAB, WQ, XQ, CSO, QOFF"
    return ("#define PHASE_NT%d_B%d(%s) \\\n    asm volatile( \\\n        %s \\\n"
            "        : %s \\\n        : %s \\\n        : %s, \"m0\", \"scc\", \"memory\")\n"
            % (nt, buf, args, body_text, ", ".join(outs), ", ".join(inp), clob))


def emit_px(buf):
    """PHASE_PX_B<buf>: one phase of the kernel variant that reads PRE-EXPANDED fills (16 columns per tile).

    A fill here is a pair of ordinary fills: 8 input channels x 16 columns = 128 slots, so that the expanded row of
    an activation code is 256 bytes, one pass over all 64 LDS banks.  The rows of a fill are built once per layer
    in memory and a phase copies the next fill (64 KiB) straight into the other LDS buffer: eight buffer loads with
    the lds modifier per wavefront, no transposition.  A lane owns two activation dwords per pixel and fill, FIRST
    and SECOND; lanes with bit 3 set hold the two swapped, and read FIRST out of the upper half of the row, so that
    the 16 lanes that share an LDS pass read 16 different 16-byte chunks.  A pixel is looked up as two units of
    eight steps (FIRST, then SECOND) that run through the same rolling window of eight reads.

    Buffer 1 lies 65536 bytes behind buffer 0, one more than the offset field of ds_read_b128 holds: its chunk
    offsets carry 15 in their low four bits and the instruction adds 65521.
    """
    rows = 8
    other = buf ^ 1

    def read(st, r, h, step):
        b = TEMP_BASE + 4 * step
        va = ADDR_BASE + (step % 4)
        st.ins("v_perm_b32 v%d, %%[%s%d], %%[ch%d%s], %%[s%d]" % (va, "fg"[h], r, h, "ab"[step >> 2], step))
        off = " offset:65521" if buf else ""
        return st.lds("ds_read_b128 v[%d:%d], v%d%s" % (b, b + 3, va, off))

    def adds(st, r, steps):
        g = steps[0] % 2
        for d in range(4):
            even = "%%[c%d_%d]" % (r, g * 8 + 2 * d)
            odd = "%%[c%d_%d]" % (r, g * 8 + 2 * d + 1)
            regs = [TEMP_BASE + 4 * step + d for step in steps]
            st.ins("v_add3_u32 %s, %s, v%d, v%d" % (even, even, regs[0], regs[1]))
            for reg in regs:
                st.ins("v_add_u32_sdwa %s, %s, v%d dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1"
                       % (odd, odd, reg))

    groups = [(0, 2), (1, 3), (4, 6), (5, 7)]

    def e_load(j):           # 1 KiB of the next fill: memory -> LDS buffer [other]
        def f(st, state):
            st.ins("s_add_u32 m0, %%[edst], %d" % (other * 65536 + j * 1024))
            st.ins("s_add_u32 %%[stmp], %%[eoff], %d" % (j * 1024))
            st.ins("buffer_load_dwordx4 %[l16], %[erc], %[stmp] offen lds")
            st.ins("s_nop 0")
        return f

    skips = [0]

    def act_load(r):         # both activation dwords of pixel r for the next fill; skipped for a pixel the wavefront
        def f(st, state):    # does not have (a gather costs the CU's address unit as much as 1 KiB of the fill)
            label = None
            if r > 0:
                label = "Lskip%d_%%=" % skips[0]
                skips[0] += 1
                st.ins("s_cmp_lt_u32 %d, %%[nr]" % r)
                st.ins("s_cbranch_scc0 %s" % label)
            st.ins("v_add_u32 v%d, %%[t%d], %%[dlf]" % (ADDR_BASE + 2, r))
            st.ins("buffer_load_dword %%[nf%d], v%d, %%[xq], %%[qoff] offen" % (r, ADDR_BASE + 2))
            st.ins("v_add_u32 v%d, %%[t%d], %%[dls]" % (ADDR_BASE + 3, r))
            st.ins("buffer_load_dword %%[ng%d], v%d, %%[xq], %%[qoff] offen" % (r, ADDR_BASE + 3))
            if label:
                st.label(label)
        return f

    aux = [e_load(j) for j in range(8)] + [act_load(r) for r in range(rows)]

    def aux_step(st, state):
        if state["pos"] < len(aux):
            aux[state["pos"]](st, state)
            state["pos"] += 1

    def aux_rest(st, state):
        while state["pos"] < len(aux):
            aux_step(st, state)

    def body(st, u, pending, with_next, state):
        """Accumulate unit u = 2 * pixel + half; with_next: refill the window with unit u + 1."""
        r, nxt = u // 2, [None] * 8
        for steps in groups:
            st.wait(max((pending[s] for s in steps), key=lambda op: st.fifo.index(op) if op in st.fifo else -1))
            adds(st, r, steps)
            for s in steps:
                if with_next:
                    nxt[s] = read(st, (u + 1) // 2, (u + 1) % 2, s)
                aux_step(st, state)
        return nxt

    main = Stream()
    main.ins("s_cmp_eq_u32 %[nr], 0")
    main.ins("s_cbranch_scc1 Lzero_%=")
    pending = [read(main, 0, 0, s) for s in range(8)]
    state = {"pos": 0}
    forks = []
    for r in range(rows):
        pending = body(main, 2 * r, pending, True, state)
        if r < rows - 1:
            main.ins("s_cmp_lt_u32 %d, %%[nr]" % (r + 1))
            main.ins("s_cbranch_scc0 Llast%d_%%=" % r)
            forks.append((r, main.fork(), list(pending), dict(state)))
            pending = body(main, 2 * r + 1, pending, True, state)
        else:
            body(main, 2 * r + 1, pending, False, state)
    aux_rest(main, state)
    main.drain()
    main.ins("s_branch Lend_%=")
    for r, st, pend, stt in forks:
        st.label("Llast%d_%%=" % r)
        body(st, 2 * r + 1, pend, False, stt)
        aux_rest(st, stt)
        st.drain()
        st.ins("s_branch Lend_%=")
    zero = Stream(main.lines)
    zero.label("Lzero_%=")
    aux_rest(zero, {"pos": 0})
    zero.drain()
    zero.label("Lend_%=")

    outs = ['[c%d_%d] "+v"(ACC[%d][%d])' % (r, i, r, i) for r in range(rows) for i in range(16)]
    outs += ['[nf%d] "=&v"(NFIRST[%d])' % (r, r) for r in range(rows)]
    outs += ['[ng%d] "=&v"(NSECOND[%d])' % (r, r) for r in range(rows)]
    outs += ['[stmp] "=&s"(STMP)']
    inp = ['[f%d] "v"(FIRST[%d])' % (r, r) for r in range(rows)]
    inp += ['[g%d] "v"(SECOND[%d])' % (r, r) for r in range(rows)]
    inp += ['[t%d] "v"(TAPOFF[%d])' % (r, r) for r in range(rows)]
    inp += ['[s%d] "v"(SEL[%d])' % (i, i) for i in range(8)]
    inp += ['[ch0a] "v"(CH[0])', '[ch0b] "v"(CH[1])', '[ch1a] "v"(CH[2])', '[ch1b] "v"(CH[3])']
    inp += ['[dlf] "v"(DLF)', '[dls] "v"(DLS)', '[l16] "v"(L16)', '[nr] "s"(NR)']
    inp += ['[edst] "s"(EDST)', '[eoff] "s"(EOFF)', '[erc] "s"(ERC)', '[xq] "s"(XQ)', '[qoff] "s"(QOFF)']
    clob = ", ".join('"v%d"' % r for r in range(ADDR_BASE, TEMP_BASE + 32))
    body_text = " \\\n        ".join(main.lines)
    args = "ACC, FIRST, SECOND, NFIRST, NSECOND, TAPOFF, SEL, CH, DLF, DLS, L16, NR, STMP, EDST, EOFF, ERC, XQ, QOFF"
    return ("#define PHASE_PX_B%d(%s) \\\n    asm volatile( \\\n        %s \\\n"
            "        : %s \\\n        : %s \\\n        : %s, \"m0\", \"scc\", \"memory\")\n"
            % (buf, args, body_text, ", ".join(outs), ", ".join(inp), clob))


# LDS control block of the kernel that reads pre-expanded fills: the last 32 bytes of the 160 KiB (the geometry slots
# of a wavefront-row that its tiles never have).  One counter per fill buffer that only grows: the eight wavefronts
# count themselves (one lane adds 1) when their share of a fill has arrived in the buffer, and again when they have
# finished reading that fill.  All eight arrivals of a fill precede the first reader, and all eight readers the
# first arrival of the next fill, so the j-th fill of a buffer is whole once the count has reached 16 j + 8 and
# the buffer free again at 16 j + 16.  EVENTS[0], EVENTS[1], ABORT.
PX_LDS_BYTES = 163840
PX_CB = PX_LDS_BYTES - 32
PX_TGT_ISSUED = 0xfffffffe     # TGT of a phase that has issued its loads,
PX_TGT_COUNTED = 0xffffffff    # and of one that has also counted their arrival
IB_STS_VM_CNT = 0x00c0000f     # the bits of the hardware register IB_STS that hold this wavefront's vmcnt
PX_FIRST = ADDR_BASE - 2       # first register the phase of the pre-expanded kernel clobbers
SCRATCH_ADDR = PX_FIRST        # address temporary of the activation loads, the polls and the count
POLL_REG = PX_FIRST + 1        # where a poll lands: EVENTS[other]


def emit_pxf():
    """PHASE_PXF: one phase of the kernel variant that reads pre-expanded fills WITHOUT a barrier between fills.

    A fill here is a pair of ordinary fills: 8 input channels x 16 columns = 128 slots, so that the expanded row of
    an activation code is 256 bytes, one pass over all 64 LDS banks.  The rows of a fill are built once per layer
    in memory and every wavefront copies its eighth of the next fill (eight buffer loads with the lds modifier)
    straight into the other LDS buffer.  A lane owns two activation dwords per pixel and fill, FIRST
    and SECOND; lanes with bit 3 set hold the two swapped, and read FIRST out of the upper half of the row, so that
    the 16 lanes that share an LDS pass read 16 different 16-byte chunks.  A pixel is looked up as two units of
    eight steps (FIRST, then SECOND) that run through the same rolling window of eight reads.

    The wavefronts of a workgroup do not meet at a barrier between fills.  The other buffer may be refilled once
    all eight wavefronts have finished the fill before this one: the phase polls EVENTS[other] when
    it starts on a pixel (one 4-byte LDS read, consumed a unit later, where the waits for the lookups have long
    covered it).  TGT carries the state.  Below 0xfffffffd it is the count EVENTS[other] has to reach: the first poll
    that finds it there issues the eight loads and sets TGT to 0xfffffffe (the caller does the same when it finds
    the buffer free before the phase).  From there every poll looks, without waiting, whether this wavefront still
    has a load in flight (its vmcnt, read from the hardware register IB_STS): the first poll that finds none adds
    the wavefront to EVENTS[other] and sets TGT to 0xffffffff.  A wavefront never waits for the loads inside the
    phase: a fill takes some 3 000 cycles to land under the lookups.  A
    phase that ends with TGT below 0xffffffff leaves what is missing to the caller.  SEEN returns the last
    EVENTS[other] a poll saw (0 without a poll): the caller may start on the next fill without a look of its own.

    One body serves both buffers.  The lookup address (buffer << 16 | row << 8 | half << 7 | chunk << 4) is one
    v_perm_b32: byte 2 <- byte 3 of the chunk register (0 or 1: the caller flips it between phases), byte 1 <- the
    activation code, byte 0 <- one of the three chunk bytes the register holds (steps 0-2, 3-5, 6-7 of a unit).  The
    LDS destination of the loads (EDST: the wavefront's eighth of the OTHER buffer) and the address of the counter
    the polls read (POLLADDR: DONE of the other buffer) are scalar operands.
    """
    rows = 8

    def address(st, r, h, step):
        va = ADDR_BASE + (step % 4)
        st.ins("v_perm_b32 v%d, %%[%s%d], %%[ch%d%s], %%[s%d]" % (va, "fg"[h], r, h, "abc"[step // 3], step))

    def read(st, r, h, step, with_address=True):
        b = TEMP_BASE + 4 * step
        va = ADDR_BASE + (step % 4)
        if with_address:
            address(st, r, h, step)
        return st.lds("ds_read_b128 v[%d:%d], v%d" % (b, b + 3, va))

    def adds(st, r, steps, halfway=None):
        """Twelve adds; no instruction reads the result of the one right before it."""
        g = steps[0] % 2
        sdwa = "v_add_u32_sdwa %s, %s, v%d dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1"
        even = lambda d: "%%[c%d_%d]" % (r, g * 8 + 2 * d)
        odd = lambda d: "%%[c%d_%d]" % (r, g * 8 + 2 * d + 1)
        reg = lambda k, d: TEMP_BASE + 4 * steps[k] + d
        for pair in ((0, 1), (2, 3)):
            if pair[0] == 2 and halfway:
                halfway()
            for d in pair:
                st.ins("v_add3_u32 %s, %s, v%d, v%d" % (even(d), even(d), reg(0, d), reg(1, d)))
            for k in range(2):
                for d in pair:
                    st.ins(sdwa % (odd(d), odd(d), reg(k, d)))

    groups = [(0, 2), (1, 3), (4, 6), (5, 7)]
    counter = [0]

    def fresh(prefix):
        counter[0] += 1
        return "%s%d_%%=" % (prefix, counter[0])

    def poll_issue(st, state):
        st.ins("v_mov_b32 v%d, %%[polladdr]" % SCRATCH_ADDR)
        state["poll"] = st.lds("ds_read_b32 v%d, v%d" % (POLL_REG, SCRATCH_ADDR))

    def poll_consume(st, state):
        st.wait(state["poll"])
        issued, end = fresh("Lis"), fresh("Lpe")
        st.ins("v_readfirstlane_b32 %%[seen], v%d" % POLL_REG)
        st.ins("s_cmp_ge_u32 %%[tgt], 0x%x" % PX_TGT_ISSUED)
        st.ins("s_cbranch_scc1 %s" % issued)
        # not yet issued: if all eight wavefronts have left the other buffer, the eight loads of 1 KiB, memory -> LDS
        st.ins("s_cmp_ge_u32 %[seen], %[tgt]")
        st.ins("s_cbranch_scc0 %s" % end)
        for j in range(8):
            st.ins("s_add_u32 m0, %%[edst], %d" % (j * 1024))
            st.ins("s_add_u32 %%[stmp], %%[eoff], %d" % (j * 1024))
            st.ins("buffer_load_dwordx4 %[l16], %[erc], %[stmp] offen lds")
            st.ins("s_nop 0")
        st.ins("s_mov_b32 %%[tgt], 0x%x" % PX_TGT_ISSUED)
        st.ins("s_branch %s" % end)
        st.label(issued)
        # issued: once none of this wavefront's loads is in flight any more, add it to EVENTS[other]
        st.ins("s_cmp_eq_u32 %[tgt], -1")
        st.ins("s_cbranch_scc1 %s" % end)
        st.ins("s_getreg_b32 %[stmp], hwreg(HW_REG_IB_STS)")
        st.ins("s_and_b32 %%[stmp], %%[stmp], 0x%x" % IB_STS_VM_CNT)
        st.ins("s_cbranch_scc1 %s" % end)
        st.ins("v_mov_b32 v%d, %%[polladdr]" % SCRATCH_ADDR)
        st.ins("v_mov_b32 v%d, 1" % POLL_REG)
        st.ins("s_mov_b64 %[sx], exec")          # one lane adds: 64 atomics on one address would hold the LDS for as many turns
        st.ins("s_mov_b64 exec, 1")
        st.ins("ds_add_u32 v%d, v%d" % (SCRATCH_ADDR, POLL_REG))   # not in the model's queue: waits stay on the safe side
        st.ins("s_mov_b64 exec, %[sx]")
        st.ins("s_mov_b32 %[tgt], -1")
        st.label(end)

    def act_load(r):         # both activation dwords of pixel r for the next fill; skipped for a pixel the wavefront
        def f(st, state):    # does not have (a gather costs the CU's address unit as much as 1 KiB of the fill)
            label = None
            if r > 0:
                label = fresh("Lskip")
                st.ins("s_cmp_lt_u32 %d, %%[nr]" % r)
                st.ins("s_cbranch_scc0 %s" % label)
            st.ins("v_add_u32 v%d, %%[t%d], %%[dlf]" % (SCRATCH_ADDR, r))
            st.ins("buffer_load_dword %%[nf%d], v%d, %%[xq], %%[qoff] offen" % (r, SCRATCH_ADDR))
            st.ins("v_add_u32 v%d, %%[t%d], %%[dls]" % (SCRATCH_ADDR, r))
            st.ins("buffer_load_dword %%[ng%d], v%d, %%[xq], %%[qoff] offen" % (r, SCRATCH_ADDR))
            if label:
                st.label(label)
        return f

    aux = [act_load(r) for r in range(rows)]

    def aux_step(st, state):
        if state["pos"] < len(aux):
            aux[state["pos"]](st, state)
            state["pos"] += 1

    def aux_rest(st, state):
        while state["pos"] < len(aux):
            aux_step(st, state)

    def body(st, u, pending, with_next, state):
        """Accumulate unit u = 2 * pixel + half; with_next: refill the window with unit u + 1."""
        r, nxt = u // 2, [None] * 8
        for gi, steps in enumerate(groups):
            st.wait(max((pending[s] for s in steps), key=lambda op: st.fifo.index(op) if op in st.fifo else -1))
            # the addresses of the next two lookups are computed in the middle of the adds, well ahead of the reads
            # that use them: a read right behind its v_perm_b32 waits for that instruction's result
            early = (lambda: [address(st, (u + 1) // 2, (u + 1) % 2, s) for s in steps]) if with_next else None
            adds(st, r, steps, early)
            if u % 2 == 1 and gi == 1:
                poll_consume(st, state)
            for s in steps:
                if with_next:
                    nxt[s] = read(st, (u + 1) // 2, (u + 1) % 2, s, with_address=False)
                aux_step(st, state)
            if u % 2 == 0 and gi == 0:
                poll_issue(st, state)
        return nxt

    main = Stream()
    main.ins("s_mov_b32 %[seen], 0")
    main.ins("s_cmp_eq_u32 %[nr], 0")
    main.ins("s_cbranch_scc1 Lzero_%=")
    pending = [read(main, 0, 0, s) for s in range(8)]
    state = {"pos": 0, "poll": None}
    forks = []
    for r in range(rows):
        pending = body(main, 2 * r, pending, True, state)
        if r < rows - 1:
            main.ins("s_cmp_lt_u32 %d, %%[nr]" % (r + 1))
            main.ins("s_cbranch_scc0 Llast%d_%%=" % r)
            forks.append((r, main.fork(), list(pending), dict(state)))
            pending = body(main, 2 * r + 1, pending, True, state)
        else:
            body(main, 2 * r + 1, pending, False, state)
    aux_rest(main, state)
    main.drain()
    main.ins("s_branch Lend_%=")
    for r, st, pend, stt in forks:
        st.label("Llast%d_%%=" % r)
        body(st, 2 * r + 1, pend, False, stt)
        aux_rest(st, stt)
        st.drain()
        st.ins("s_branch Lend_%=")
    zero = Stream(main.lines)
    zero.label("Lzero_%=")
    aux_rest(zero, {"pos": 0, "poll": None})
    zero.drain()
    zero.label("Lend_%=")

    outs = ['[c%d_%d] "+v"(ACC[%d][%d])' % (r, i, r, i) for r in range(rows) for i in range(16)]
    outs += ['[nf%d] "=&v"(NFIRST[%d])' % (r, r) for r in range(rows)]
    outs += ['[ng%d] "=&v"(NSECOND[%d])' % (r, r) for r in range(rows)]
    outs += ['[stmp] "=&s"(STMP)', '[tgt] "+s"(TGT)', '[seen] "=&s"(SEEN)', '[sx] "=&s"(SX)']
    inp = ['[f%d] "v"(FIRST[%d])' % (r, r) for r in range(rows)]
    inp += ['[g%d] "v"(SECOND[%d])' % (r, r) for r in range(rows)]
    inp += ['[t%d] "v"(TAPOFF[%d])' % (r, r) for r in range(rows)]
    inp += ['[s%d] "v"(SEL[%d])' % (i, i) for i in range(8)]
    inp += ['[ch%d%s] "v"(CH[%d])' % (h, "abc"[i], 3 * h + i) for h in range(2) for i in range(3)]
    inp += ['[dlf] "v"(DLF)', '[dls] "v"(DLS)', '[l16] "v"(L16)', '[nr] "s"(NR)', '[polladdr] "s"(POLLADDR)']
    inp += ['[edst] "s"(EDST)', '[eoff] "s"(EOFF)', '[erc] "s"(ERC)', '[xq] "s"(XQ)', '[qoff] "s"(QOFF)']
    clob = ", ".join('"v%d"' % r for r in range(PX_FIRST, TEMP_BASE + 32))
    body_text = " \\\n        ".join(main.lines)
    args = ("ACC, FIRST, SECOND, NFIRST, NSECOND, TAPOFF, SEL, CH, DLF, DLS, L16, NR, STMP, SX, TGT, SEEN, POLLADDR, EDST, "
            "EOFF, ERC, XQ, QOFF")
    return ("#define PHASE_PXF(%s) \\\n    asm volatile( \\\n        %s \\\n"
            "        : %s \\\n        : %s \\\n        : %s, \"m0\", \"scc\", \"memory\")\n"
            % (args, body_text, ", ".join(outs), ", ".join(inp), clob))


if __name__ == "__main__":
    print("// Generated by gen_lookup_asm.py -- do not edit.")
    for nt in (16, 32, 64):
        for buf in (0, 1):
            print(emit(nt, buf))
    for buf in (0, 1):
        print(emit_px(buf))
    print(emit_pxf())
