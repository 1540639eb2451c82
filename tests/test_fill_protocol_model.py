"""The LUT-GEMM kernel without barriers (lutgemm_pxf_kernel in tf-approximate_amd/csrc/lutgemm_px_kernel.hip) lets the
eight wavefronts of a workgroup stream through the fills g = 0, 1, 2, ... (fill g in LDS buffer g & 1) held together
only by one counter per buffer that never decreases: each wavefront adds one when its eighth of a fill has landed in the
buffer and one when it has finished reading that fill, so buffer b's fill j is whole at 8 (2 j + 1) and free again at
8 (2 j + 2).

This test runs that protocol, as the kernel's comments state it, as eight co-operating state machines under random
schedules, with the copies landing at random times, and checks what the counters are there to guarantee:
  * nobody reads a fill before all eight eighths have landed;
  * nobody copies into a buffer that some wavefront still reads (or has yet to read);
  * a wavefront that skips its own wait because the polls of the phase before saw the fill whole is right to do so;
  * every wavefront finishes, no wavefront is ever more than one fill ahead of the slowest, and the counters end at
    8 x (arrivals + readers);
  * a wait that runs out ends every wavefront (no one spins for ever on a counter that will not move).
The same checker must fail when a threshold is off by one event, so that it is seen to look."""
import random

import pytest

WAVES = 8
ISSUED, COUNTED = 0xfffffffe, 0xffffffff


class Violation(AssertionError):
    pass


class Workgroup:
    def __init__(self, fills, pixels, rng, whole=lambda j: WAVES * (2 * j + 1), free=lambda j: WAVES * (2 * j + 2),
                 spin_limit=10 ** 9, stuck_wave=None):
        self.fills, self.pixels, self.rng = fills, pixels, rng
        self.whole, self.free = whole, free
        self.events = [0, 0]
        self.abort = False
        self.spin_limit = spin_limit
        self.stuck_wave = stuck_wave
        self.landed = {}                       # fill -> set of wavefronts whose eighth is in LDS
        self.in_flight = []                    # (wavefront, fill) copies issued and not landed
        self.finished_fill = [-1] * WAVES      # last fill a wavefront is done reading
        self.reading = [None] * WAVES
        self.gave_up = []

    # ---- what the hardware does on its own ----
    def land_some(self):
        keep = []
        for w, fill in self.in_flight:
            if self.rng.random() < 0.3:
                self.landed.setdefault(fill, set()).add(w)
            else:
                keep.append((w, fill))
        self.in_flight = keep

    def land_all_of(self, w):                  # s_waitcnt vmcnt(0)
        for ww, fill in self.in_flight:
            if ww == w:
                self.landed.setdefault(fill, set()).add(w)
        self.in_flight = [(ww, f) for ww, f in self.in_flight if ww != w]

    def has_in_flight(self, w):
        return any(ww == w for ww, _ in self.in_flight)

    # ---- the checks ----
    def copy(self, w, fill):
        if fill >= 2:
            for other in range(WAVES):
                if self.finished_fill[other] < fill - 2:
                    raise Violation("wavefront %d copies fill %d over fill %d, which wavefront %d has not finished"
                                    % (w, fill, fill - 2, other))
        self.in_flight.append((w, fill))

    def begin_reading(self, w, fill):
        if len(self.landed.get(fill, ())) != WAVES:
            raise Violation("wavefront %d reads fill %d with %d eighths landed"
                            % (w, fill, len(self.landed.get(fill, ()))))
        self.reading[w] = fill
        if fill - (min(self.finished_fill) + 1) > 1:
            raise Violation("wavefront %d is more than a fill ahead" % w)

    # ---- one wavefront ----
    def wait_for(self, w, buffer, target):
        polls = 0
        while True:
            ev = list(self.events)
            if ev[buffer] >= target:
                return ev
            if polls >= self.spin_limit or self.abort:
                return None
            polls += 1
            yield

    def wave(self, w):
        self.copy(w, 0)
        yield
        self.land_all_of(w)
        if w != self.stuck_wave:               # a wavefront that never counts: every wait on fill 0 must run out
            self.events[0] += 1
        seen = 0
        for g in range(self.fills):
            buf, other = g & 1, (g & 1) ^ 1
            loads = g + 1 < self.fills
            tgt = COUNTED if not loads else 0 if g == 0 else self.free((g - 1) >> 1)
            if seen < self.whole(g >> 1):
                ev = yield from self.wait_for(w, buf, self.whole(g >> 1))
                if ev is None:
                    self.abort = True
                    self.gave_up.append(w)
                    return
                if loads and ev[other] >= tgt:
                    self.copy(w, g + 1)
                    tgt = ISSUED
            self.begin_reading(w, g)
            seen = 0
            for _ in range(self.pixels[w]):    # the phase body: one poll per pixel, lookups in between
                yield
                if len(self.landed.get(g, ())) != WAVES:
                    raise Violation("fill %d lost an eighth under wavefront %d" % (g, w))
                seen = self.events[other]
                if tgt < ISSUED:
                    if seen >= tgt:
                        self.copy(w, g + 1)
                        tgt = ISSUED
                elif tgt == ISSUED and not self.has_in_flight(w):
                    self.events[other] += 1
                    tgt = COUNTED
            yield
            if tgt < ISSUED:
                ev = yield from self.wait_for(w, other, tgt)
                if ev is None:
                    self.abort = True
                    self.gave_up.append(w)
                    return
                self.copy(w, g + 1)
                tgt = ISSUED
            self.land_all_of(w)                # the body, or the wait behind it, ends with vmcnt(0)
            if tgt != COUNTED:
                self.events[other] += 1
            self.reading[w] = None
            self.finished_fill[w] = g
            self.events[buf] += 1

    def run(self, bias=None):
        waves = {w: self.wave(w) for w in range(WAVES)}
        steps = 0
        while waves:
            if bias and self.rng.random() < 0.8:
                pool = [w for w in waves if w in bias] or list(waves)
            else:
                pool = list(waves)
            w = self.rng.choice(pool)
            try:
                next(waves[w])
            except StopIteration:
                del waves[w]
            self.land_some()
            steps += 1
            assert steps < 10 ** 7, "the workgroup does not finish"
        return steps


def _pixels(rng, kind):
    if kind == "full":
        return [8] * WAVES
    if kind == "empty tail":                   # wavefronts without a pixel never poll inside the body
        return [8, 8, 8, 1, 0, 0, 0, 0]
    return [rng.randrange(0, 9) for _ in range(WAVES)]


@pytest.mark.parametrize("kind", ["full", "empty tail", "ragged"])
@pytest.mark.parametrize("fills", [1, 2, 3, 8, 17])
def test_counters_keep_readers_and_copies_apart(fills, kind):
    for seed in range(40):
        rng = random.Random(1000 * fills + seed)
        wg = Workgroup(fills, _pixels(rng, kind), rng)
        # some schedules favour a few wavefronts, so that they run as far ahead as the protocol lets them
        wg.run(bias=None if seed % 2 else set(rng.sample(range(WAVES), 3)))
        arrivals = [len(range(b, fills, 2)) for b in range(2)]
        assert wg.events == [2 * WAVES * arrivals[0], 2 * WAVES * arrivals[1]]
        assert wg.finished_fill == [fills - 1] * WAVES and not wg.in_flight and not wg.gave_up


@pytest.mark.parametrize("broken", ["whole one event early", "free one event early"])
def test_the_checker_notices_a_threshold_that_is_off_by_one_event(broken):
    kw = {"whole": lambda j: WAVES * (2 * j + 1) - 1} if broken.startswith("whole") \
        else {"free": lambda j: WAVES * (2 * j + 2) - 1}
    caught = 0
    for seed in range(60):
        rng = random.Random(seed)
        wg = Workgroup(9, [8] * WAVES, rng, **kw)
        try:
            wg.run(bias=set(rng.sample(range(WAVES), 3)))
        except Violation:
            caught += 1
    assert caught > 0


def test_a_wait_that_runs_out_ends_every_wavefront():
    """One wavefront never counts its part of the first fill (as if its copy never landed): the others' waits run out
    after spin_limit polls, the first one raises ABORT, and everybody leaves instead of spinning."""
    for seed in range(10):
        rng = random.Random(seed)
        wg = Workgroup(6, [8] * WAVES, rng, spin_limit=50, stuck_wave=seed % WAVES)
        wg.run()
        assert sorted(wg.gave_up) == list(range(WAVES))
        assert wg.finished_fill == [-1] * WAVES
