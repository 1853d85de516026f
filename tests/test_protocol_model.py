"""Discrete-event model of the producer/consumer counter protocol (CPU only).

The GPU kernel synchronises producer and consumer waves through monotonically increasing counters per
stage: full[unit] (+1 per producer wave of the operand once the rows of that unit have landed) and
empty[unit] (+1 per consumer wave that has finished reading them). Which wave waits for / signals
which counter, and with which expected value, is restated here from the kernel's rules for the three
granularities (tile, wave tile with bar_steps_a/b, 16-row block with bar_steps_a/b); the reference's
cuda::barrier protocol it re-expresses is matmul_shmem_tc_async_opt_port_2.cu:212-305 (producers) and
:495-600 (consumers). The model runs every wave as a generator under a random scheduler and checks the
two properties no numeric test can see directly:

  * safety: a consumer only reads a row block of a stage that holds the segment it is about to multiply,
    and a producer only overwrites a row block after every reader of the previous fill has released it;
  * liveness: whatever the interleaving, all waves finish (no deadlock).
"""
import itertools
import random

import pytest

TILE_MODE, WAVE_MODE, ACC_MODE = 0, 1, 2


class Model:
    def __init__(self, mode, cw, pa, pb, sa, sb, stages, nseg, ntiles, wtr, wtc, rng):
        self.mode, self.cw, self.pa, self.pb, self.sa, self.sb = mode, cw, pa, pb, sa, sb
        self.S, self.nseg, self.ntiles, self.wtr, self.wtc, self.rng = stages, nseg, ntiles, wtr, wtc, rng
        self.rows_a, self.rows_b = cw // 2, 2          # wave-tile rows of A, wave-tile columns of Bt
        if mode == TILE_MODE:
            self.ua = self.ub = 1
        elif mode == WAVE_MODE:
            self.ua, self.ub = sa + 1, sb + 1
        else:
            self.ua, self.ub = self.rows_a * (sa + 1), self.rows_b * (sb + 1)
        z = lambda n: [[0] * n for _ in range(stages)]
        self.full = {"A": z(self.ua), "B": z(self.ub)}
        self.empty = {"A": z(self.ua), "B": z(self.ub)}
        # ground truth per (operand, stage, 16-row block): which global segment each producer wave last wrote.
        # Every block is read by its readers in every segment, so both a read before the data has landed
        # (block still holds an older segment) and an overwrite before the last read (block already holds
        # a newer one) show up as a read of the wrong segment.
        nblk = {"A": self.rows_a * wtr, "B": self.rows_b * wtc}
        self.nblk = nblk
        self.holds = {op: [[[-1] * (pa if op == "A" else pb) for _ in range(nblk[op])] for _ in range(stages)] for op in "AB"}
        self.errors = []

    # ---- row-block units -------------------------------------------------------------------------------
    def blocks_of_unit(self, op, blk):
        """16-row blocks one producer 'row block' covers, by granularity."""
        wt = self.wtr if op == "A" else self.wtc
        if self.mode == TILE_MODE:
            return range(self.nblk[op])
        if self.mode == WAVE_MODE:
            return range(blk * wt, (blk + 1) * wt)
        return range(blk, blk + 1)

    def readers_per_block(self, op):
        return 2 if op == "A" else self.cw // 2

    # ---- producer wave q of operand op ---------------------------------------------------------------------
    def producer(self, op, q):
        px = self.pa if op == "A" else self.pb
        s_own, s_oth = (self.sa, self.sb) if op == "A" else (self.sb, self.sa)
        oth_max = 2 if op == "A" else self.cw // 2
        wt = self.wtr if op == "A" else self.wtc
        nunits = 1 if self.mode == TILE_MODE else (self.rows_a if op == "A" else self.rows_b) * (1 if self.mode == WAVE_MODE else wt)
        nres = self.cw - self.sa * self.sb
        g = 0
        for tile in range(self.ntiles):
            for seg in range(self.nseg):
                stage, fill = g % self.S, g // self.S
                E, F = self.empty[op][stage], self.full[op][stage]
                for blk in range(nunits):
                    # ---- waits (expected value = readers x fill)
                    waits = []
                    if self.mode == TILE_MODE:
                        waits.append((0, self.cw * fill))
                    elif self.mode == WAVE_MODE:
                        first_has_res = s_own == 0 or s_oth < oth_max
                        if blk == 0 and first_has_res and nres > 0:
                            waits.append((s_own, nres * fill))
                        if blk < s_own and s_oth > 0:
                            waits.append((blk, s_oth * fill))
                        elif blk == s_own and not first_has_res and nres > 0:
                            waits.append((s_own, nres * fill))
                    else:
                        unit, sub = divmod(blk, wt)
                        if sub <= s_own:
                            waits.append((unit * (s_own + 1) + sub, self.readers_per_block(op) * fill))
                    for idx, target in waits:
                        while E[idx] < target:
                            yield
                    # ---- "load": every 16-row block of this unit now holds segment g (this wave's share)
                    for b in self.blocks_of_unit(op, blk):
                        self.holds[op][stage][b][q] = g
                    yield
                    # ---- signals
                    if self.mode == TILE_MODE:
                        F[0] += 1
                    elif self.mode == WAVE_MODE:
                        if blk < s_own:
                            F[blk] += 1
                        if blk == nunits - 1:
                            F[s_own] += 1
                    else:
                        unit, sub = divmod(blk, wt)
                        if sub < s_own:
                            F[unit * (s_own + 1) + sub] += 1
                        elif sub == wt - 1:
                            F[unit * (s_own + 1) + s_own] += 1
                    yield
                g += 1

    # ---- consumer wave cw ---------------------------------------------------------------------------------
    def read(self, op, stage, b, g):
        for q, h in enumerate(self.holds[op][stage][b]):
            if h != g:
                self.errors.append("consumer read %s stage %d block %d expecting segment %d, producer %d had written %d" % (op, stage, b, g, q, h))

    def consumer(self, w):
        R, Cc = divmod(w, 2)
        pa, pb = self.pa, self.pb
        g = 0
        for tile in range(self.ntiles):
            for seg in range(self.nseg):
                stage, fill = g % self.S, g // self.S
                FA, FB, EA, EB = self.full["A"][stage], self.full["B"][stage], self.empty["A"][stage], self.empty["B"][stage]
                a_blocks = range(R * self.wtr, (R + 1) * self.wtr)
                b_blocks = range(Cc * self.wtc, (Cc + 1) * self.wtc)
                if self.mode != ACC_MODE:
                    individual = self.mode == WAVE_MODE and R < self.sa and Cc < self.sb
                    ia = (R if individual else self.sa) if self.mode == WAVE_MODE else 0
                    ib = (Cc if individual else self.sb) if self.mode == WAVE_MODE else 0
                    while FA[ia] < pa * (fill + 1):
                        yield
                    while FB[ib] < pb * (fill + 1):
                        yield
                    for b in a_blocks:
                        self.read("A", stage, b, g)
                    for b in b_blocks:
                        self.read("B", stage, b, g)
                    yield
                    EA[ia] += 1
                    EB[ib] += 1
                else:
                    sa, sb = self.sa, self.sb
                    fa0, fb0 = R * (sa + 1), Cc * (sb + 1)
                    a_waited = -1
                    for i in range(self.wtr):                      # phase 1: first sb columns
                        for j in range(min(sb, self.wtc)):
                            ai = min(i, sa)
                            if ai > a_waited:
                                while FA[fa0 + ai] < pa * (fill + 1):
                                    yield
                                a_waited = ai
                            if i == 0:
                                while FB[fb0 + j] < pb * (fill + 1):
                                    yield
                            self.read("A", stage, R * self.wtr + i, g)
                            self.read("B", stage, Cc * self.wtc + j, g)
                            yield
                            if i == self.wtr - 1:
                                EB[fb0 + j] += 1
                    while FB[fb0 + sb] < pb * (fill + 1):            # phase 2: residual columns
                        yield
                    for i in range(self.wtr):
                        ai = min(i, sa)
                        if ai > a_waited:
                            while FA[fa0 + ai] < pa * (fill + 1):
                                yield
                            a_waited = ai
                        self.read("A", stage, R * self.wtr + i, g)
                        for j in range(sb, self.wtc):
                            self.read("B", stage, Cc * self.wtc + j, g)
                        yield
                        if i < sa:
                            EA[fa0 + i] += 1
                        if i == self.wtr - 1:
                            EA[fa0 + sa] += 1
                            EB[fb0 + sb] += 1
                g += 1

    # ---- run ------------------------------------------------------------------------------------------------
    def run(self):
        waves = [self.producer("A", q) for q in range(self.pa)] + [self.producer("B", q) for q in range(self.pb)]
        waves += [self.consumer(w) for w in range(self.cw)]
        alive = list(range(len(waves)))
        idle_rounds = 0
        snapshot = None
        while alive:
            i = self.rng.choice(alive)
            try:
                next(waves[i])
            except StopIteration:
                alive.remove(i)
            state = (tuple(map(tuple, self.full["A"])), tuple(map(tuple, self.full["B"])),
                     tuple(map(tuple, self.empty["A"])), tuple(map(tuple, self.empty["B"])), len(alive))
            idle_rounds = idle_rounds + 1 if state == snapshot else 0
            snapshot = state
            if idle_rounds > 2000 * len(waves):
                return "deadlock with %d waves alive" % len(alive)
        return None


def shapes(tile, cw):
    wtr = tile // (cw // 2) // 16
    wtc = tile // 2 // 16
    return wtr, wtc


def check(mode, tile, cw, p, sa, sb, stages, nseg, ntiles, seed):
    wtr, wtc = shapes(tile, cw)
    m = Model(mode, cw, p // 2, p - p // 2, sa, sb, stages, nseg, ntiles, wtr, wtc, random.Random(seed))
    dead = m.run()
    assert dead is None, (mode, tile, cw, p, sa, sb, stages, dead)
    assert not m.errors, (mode, tile, cw, p, sa, sb, stages, m.errors[:3])


@pytest.mark.parametrize("cw,p", [(4, 2), (8, 2), (8, 4), (4, 8)])
def test_tile_granularity(cw, p):
    for stages, nseg in ((1, 5), (2, 7), (4, 3), (3, 9)):
        check(TILE_MODE, 128, cw, p, 0, 0, stages, nseg, 2, 1000 + stages)


@pytest.mark.parametrize("cw", [4, 8])
def test_wave_tile_granularity_all_bar_steps(cw):
    for sa, sb in itertools.product(range(cw // 2 + 1), range(3)):
        for stages, p in ((1, 2), (2, 4), (3, 2)):
            check(WAVE_MODE, 128, cw, p, sa, sb, stages, 6, 2, 7 * sa + sb + stages)


@pytest.mark.parametrize("tile,cw", [(64, 4), (128, 4), (128, 8), (256, 8)])
def test_block_granularity_all_bar_steps(tile, cw):
    wtr, wtc = shapes(tile, cw)
    for sa, sb in itertools.product(sorted({0, wtr // 2, wtr - 1}), sorted({0, wtc // 2, wtc - 1})):
        for stages, p in ((1, 2), (2, 4)):
            check(ACC_MODE, tile, cw, p, sa, sb, stages, 4, 2, 31 * sa + sb + stages)


def test_model_detects_a_broken_protocol():
    # sanity of the checker itself: producers that do not wait for the 'empty' counters (pre-loaded here)
    # run ahead and overwrite segments before they are read - the model must notice
    wtr, wtc = shapes(128, 4)
    m = Model(TILE_MODE, 4, 1, 1, 0, 0, 1, 6, 1, wtr, wtc, random.Random(5))
    for s in range(m.S):
        m.empty["A"][s][0] = m.empty["B"][s][0] = 10 ** 6
    for pw in (m.producer("A", 0), m.producer("B", 0)):
        for _ in pw:
            pass
    for cwv in [m.consumer(w) for w in range(4)]:
        for _ in itertools.islice(cwv, 50):
            pass
    assert m.errors
    # and a consumer that expects fewer producer signals than there are producers reads too early
    m = Model(TILE_MODE, 4, 2, 2, 0, 0, 2, 6, 1, wtr, wtc, random.Random(6))
    m.pa = m.pb = 1   # consumers wait for one signal per fill while two producer waves write
    waves = [Model.producer(m, "A", q) for q in range(2)] + [Model.producer(m, "B", q) for q in range(2)] + [m.consumer(w) for w in range(4)]
    rng, alive = random.Random(7), list(range(len(waves)))
    for _ in range(20000):
        if not alive:
            break
        i = rng.choice(alive)
        try:
            next(waves[i])
        except StopIteration:
            alive.remove(i)
    assert m.errors


# ---- the fused variant: workgroup barrier per segment, every wave loads its share -----------------------
class FusedModel:
    """Waves of the fused kernel. A wave's loads land in issue order after arbitrary delays; at the last
    k-step of segment G a wave waits for its own loads of G+1, meets the others at the barrier, issues its
    share of segment G+S into the stage of G and reads fragments of G+1 (any wave's share)."""

    def __init__(self, waves, stages, total, rng):
        self.n, self.S, self.total, self.rng = waves, stages, total, rng
        self.holds = [[-1] * waves for _ in range(stages)]        # per stage, per loading wave: segment landed
        self.inflight = [[] for _ in range(waves)]                 # per wave: FIFO of (stage, segment)
        self.arrived, self.generation = 0, 0
        self.errors = []

    def land_some(self):
        w = self.rng.randrange(self.n)
        if self.inflight[w]:
            stage, seg = self.inflight[w].pop(0)
            self.holds[stage][w] = seg

    def wave(self, w):
        S, total = self.S, self.total
        issued = 0
        for _ in range(min(S, total)):                             # prologue fills every stage
            self.inflight[w].append((issued % S, issued))
            issued += 1
        def landed(x):                                             # own loads of segment x have landed
            return all(seg > x for _, seg in self.inflight[w])
        def barrier():
            gen = self.generation
            self.arrived += 1
            if self.arrived == self.n:
                self.arrived = 0
                self.generation += 1
            while self.generation == gen:
                yield
        while not landed(0):
            yield
        yield from barrier()
        self.read(0, 0)
        for G in range(total):
            if G + 1 < total:
                while not landed(G + 1):
                    yield
                yield from barrier()
                if issued < total:
                    self.inflight[w].append((issued % S, issued))   # into the stage of segment G
                    issued += 1
                yield
                self.read((G + 1) % S, G + 1)
            yield

    def read(self, stage, seg):
        for w, h in enumerate(self.holds[stage]):
            if h != seg:
                self.errors.append("read stage %d expecting segment %d, wave %d's share holds %d" % (stage, seg, w, h))

    def run(self):
        gens = [self.wave(w) for w in range(self.n)]
        alive = list(range(self.n))
        steps = 0
        while alive:
            steps += 1
            if steps > 400000:
                return "deadlock"
            if self.rng.random() < 0.3:
                self.land_some()
                continue
            i = self.rng.choice(alive)
            try:
                next(gens[i])
            except StopIteration:
                alive.remove(i)
        return None


@pytest.mark.parametrize("waves", [4, 8])
def test_fused_barrier_protocol(waves):
    for stages, total in ((2, 9), (3, 10), (5, 4), (4, 1), (2, 2)):
        m = FusedModel(waves, stages, total, random.Random(100 * stages + total))
        assert m.run() is None
        assert not m.errors, m.errors[:3]


def test_fused_model_detects_a_missing_landing_wait():
    # sanity of the checker: hide the in-flight queues from the landing check, so no wave waits for its loads
    m = FusedModel(4, 2, 8, random.Random(3))
    m.inflight = [_AlwaysEmptyView() for _ in range(4)]
    m.run()
    assert m.errors


class _AlwaysEmptyView(list):
    """In-flight queue whose contents the landing check cannot see (iteration yields nothing)."""
    def __iter__(self):
        return iter(())


# ---- the straight-line kernel: five quarters, pair fetch, counted waits --------------------------------
class StreamModel:
    """Waves of the straight-line 256 x 256 kernel, restated from its schedule. Every wave keeps one queue
    of vector memory operations that complete in issue order (loads and the epilogue's stores alike) and
    waits with `outstanding <= immediate`, exactly as `s_waitcnt vmcnt` does. Loop body = even and odd
    k-step of a work item's K range; in the even k-step a wave issues its two A load pairs of the body two
    ahead, in the odd one the two Bt pairs; each pair is two loads (the halves of a line) into quarters
    (j + 4) % 5 and j % 5 of the even k-step j. The odd k-step waits with immediate 4 (+ 32 behind an
    epilogue without C reads); every k-step has one barrier, behind it the fragments of the next k-step
    are read. In the other schedule (odd_only) the even k-step has neither barrier nor loads, the odd one
    issues all four pairs and waits with immediate 0 (+ 32). Checked: a read finds every wave's share of the expected k-step in the quarter (nothing
    late, nothing overwritten early), and all waves finish."""

    LOADS_PER_KSTEP = 4
    STORES = 32

    def __init__(self, waves, bodies_per_item, items, rng, imm=4, imm_stores=36, count_stores=True, completion_rate=0.35, slow_wave=None,
                 odd_only=False, bt_pairs=2, stores=32):
        self.n, self.nb, self.items, self.rng = waves, bodies_per_item, items, rng
        self.completion_rate = completion_rate                       # how eagerly the memory system answers
        self.slow_wave = slow_wave                                   # a wave whose operations complete 50 times more rarely
        self.odd_only = odd_only                                     # no barrier and no loads in the even k-step (immediates 0 / 32)
        self.imm, self.imm_stores, self.count_stores = imm, imm_stores, count_stores
        self.bt_pairs, self.stores = bt_pairs, stores                # 256 x 128 tiles: one load pair of Bt per wave and body, 16 stores per epilogue
        self.slots = 2 + bt_pairs
        self.total = 2 * bodies_per_item * items                     # k-steps in the stream
        # per quarter and wave, per load of a k-step (A rows 16w.., A rows 16(w+8).., Bt likewise): k-step it holds
        self.holds = [[[-1] * self.slots for _ in range(waves)] for _ in range(5)]
        self.queue = [[] for _ in range(waves)]                       # per wave: FIFO of ops
        self.arrived, self.generation = 0, 0
        self.errors = []

    def complete_some(self):
        w = self.rng.randrange(self.n)
        if w == self.slow_wave and self.rng.random() > 0.02:
            return
        if self.queue[w]:
            op = self.queue[w].pop(0)
            if op[0] == "load":
                _, quarter, slot, kstep = op
                self.holds[quarter][w][slot] = kstep

    def read(self, quarter, kstep):
        for w in range(self.n):
            if self.holds[quarter][w] != [kstep] * self.slots:
                self.errors.append("k-step %d read from quarter %d: wave %d's share holds %s" % (kstep, quarter, w, self.holds[quarter][w]))

    def issue_pairs(self, w, operand, even_kstep, body_kstep):
        # two pairs = four loads of the body whose even k-step is body_kstep, issued in (or before) the body
        # of even k-step even_kstep, which fixes the quarters: lo halves -> body_kstep % 5, hi halves -> + 1
        for pair in range(2 if operand == 0 else self.bt_pairs):
            for half in range(2):
                k = body_kstep + half
                self.queue[w].append(("load", k % 5, 2 * operand + pair, k if k < self.total else -2))

    def wave(self, w):
        def barrier():
            gen = self.generation
            self.arrived += 1
            if self.arrived == self.n:
                self.arrived = 0
                self.generation += 1
            while self.generation == gen:
                yield
        def wait(imm):
            while len(self.queue[w]) > imm:
                yield
        # prologue: both operands of bodies 0 and 1, then k-step 0 in registers
        for body in (0, 1):
            for operand in (0, 1):
                self.issue_pairs(w, operand, 0, 2 * body)
        yield from wait(2 * self.slots)
        yield from barrier()
        self.read(0, 0)
        stores_in_flight = False
        for j in range(0, self.total, 2):
            # even k-step j
            if not self.odd_only:
                yield from barrier()
            yield
            self.read((j + 1) % 5, j + 1)
            if not self.odd_only:
                self.issue_pairs(w, 0, j, j + 4)
            yield
            # odd k-step j + 1
            yield from wait(self.imm_stores if stores_in_flight else self.imm)
            yield from barrier()
            yield
            if j + 2 < self.total:
                self.read((j + 2) % 5, j + 2)
            if self.odd_only:
                self.issue_pairs(w, 0, j, j + 4)
            self.issue_pairs(w, 1, j, j + 4)
            stores_in_flight = False
            if (j + 2) % (2 * self.nb) == 0:                          # the item ends: epilogue
                for _ in range(self.stores):
                    self.queue[w].append(("store",))
                stores_in_flight = self.count_stores
            yield

    def run(self):
        gens = [self.wave(w) for w in range(self.n)]
        alive = list(range(self.n))
        steps = 0
        while alive:
            steps += 1
            if steps > 8000000:
                return "deadlock"
            if self.rng.random() < self.completion_rate:
                self.complete_some()
                continue
            i = self.rng.choice(alive)
            try:
                next(gens[i])
            except StopIteration:
                alive.remove(i)
        return None


# the two schedules of the kernel: a barrier in every k-step (immediates 4 / 36), or in the odd k-step only (0 / 32)
SCHEDULES = {"barrier_every_kstep": dict(imm=4, imm_stores=36, odd_only=False), "odd_only": dict(imm=0, imm_stores=32, odd_only=True),
             # 256 x 128 tiles: six loads per body (A's four in the even k-step as before, Bt's two in the odd one), 16 stores per epilogue
             "half_width_barrier_every_kstep": dict(imm=4, imm_stores=20, odd_only=False, bt_pairs=1, stores=16),
             "half_width_odd_only": dict(imm=0, imm_stores=16, odd_only=True, bt_pairs=1, stores=16),
             # 256 x 192 tiles: eight loads per body in every wave (the second Bt pair of waves 4 .. 7 fetches nothing but is issued
             # and completes in order like any other), 24 stores per epilogue
             "three_quarter_width_barrier_every_kstep": dict(imm=4, imm_stores=28, odd_only=False, bt_pairs=2, stores=24),
             "three_quarter_width_odd_only": dict(imm=0, imm_stores=24, odd_only=True, bt_pairs=2, stores=24),
             # an epilogue that issues MORE stores than the landing wait counts is safe (the wait only gets longer): 16-bit output
             # off the 16-byte boundaries goes through the per-block epilogue (one store per accumulator block, 32) and element-wise
             # epilogues issue several stores per block, while the wait counts the 32 of the whole-line form
             "per_block_epilogue": dict(imm=4, imm_stores=36, odd_only=False, stores=32),
             "element_wise_epilogue": dict(imm=4, imm_stores=36, odd_only=False, stores=48)}


@pytest.mark.parametrize("schedule", sorted(SCHEDULES))
@pytest.mark.parametrize("bodies,items", [(1, 1), (1, 5), (2, 3), (3, 2), (7, 2), (16, 1)])
def test_stream_schedule(bodies, items, schedule):
    kw = SCHEDULES[schedule]
    for seed, rate, slow in ((0, 0.35, None), (1, 0.35, 3), (2, 0.05, None), (3, 0.05, 6)):   # eager, sluggish, one starved wave
        m = StreamModel(8, bodies, items, random.Random(1000 * bodies + 10 * items + seed), completion_rate=rate, slow_wave=slow, **kw)
        assert m.run() is None
        assert not m.errors, m.errors[:3]
    # with C reads in the epilogue the kernel does not count the stores: the stricter immediate is also safe
    m = StreamModel(8, bodies, items, random.Random(7), count_stores=False, **kw)
    assert m.run() is None and not m.errors


def test_stream_model_detects_wrong_immediates():
    # sanity of the checker: one operation too many allowed in flight, with and without the stores
    caught = 0
    for seed in range(20):
        m = StreamModel(8, 3, 3, random.Random(seed), imm=5, imm_stores=37, completion_rate=0.3, slow_wave=seed % 8)
        m.run()
        caught += bool(m.errors)
    assert caught > 0
    caught = 0
    for seed in range(20):
        m = StreamModel(8, 1, 6, random.Random(seed), imm=4, imm_stores=37, completion_rate=0.3, slow_wave=seed % 8)
        m.run()
        caught += bool(m.errors)
    assert caught > 0
    for imm, imm_stores in ((1, 33), (0, 33)):
        caught = 0
        for seed in range(20):
            m = StreamModel(8, 2, 4, random.Random(seed), imm=imm, imm_stores=imm_stores, completion_rate=0.3, slow_wave=seed % 8, odd_only=True)
            m.run()
            caught += bool(m.errors)
        assert caught > 0
    # an epilogue that issues FEWER stores than the wait counts (what the kernel's static_assert on the per-block path rules out)
    caught = 0
    for seed in range(20):
        m = StreamModel(8, 1, 6, random.Random(seed), imm=4, imm_stores=36, completion_rate=0.3, slow_wave=seed % 8, stores=16)
        m.run()
        caught += bool(m.errors)
    assert caught > 0
    # 256 x 128 tiles (16 stores per epilogue): one store too many allowed in flight, and the full-width immediate
    for imm_stores in (21, 36):
        caught = 0
        for seed in range(20):
            m = StreamModel(8, 1, 6, random.Random(seed), imm=4, imm_stores=imm_stores, completion_rate=0.3, slow_wave=seed % 8, bt_pairs=1, stores=16)
            m.run()
            caught += bool(m.errors)
        assert caught > 0
