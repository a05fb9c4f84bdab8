"""CPU model of the ticket / flag-chain protocol of csrc/ssd_chain.hip (the replacement of the reference's global
barrier, kernels/fused_globalbar.py:130-137, and of its completion counters and throttle semaphore,
kernels/fused_concurrent.py:81-84, 141, 205-208).

The model keeps what the argument for the kernel rests on and nothing else: a ticket counter, chunk-major work items
(ticket t -> chunks R (t / units) .., unit t % units), workgroups that work through their tickets in the order they
drew them and draw one ticket per item (the second during the first chunk of the first item, the third during its
second chunk), a flag per (unit, chunk) raised after the item's last state is stored, a bounded wait that gives up,
reports and still raises its flag, and the cut of an item at a sequence start.  Workgroups are advanced one event at a
time by an adversarial (seeded random) scheduler with a limit on how many may be resident, down to one -- the hardware
promises nothing about residency.  Checked: every launch drains, every passed state equals the serial recurrence
(ssd_state_passing.py:69-84 on scalars), no wait gives up when the limit is generous, and a limit of one poll is
reported while the launch still drains.  A workspace may be kept from launch to launch without clearing: flags hold the
epoch they were raised in, ticket counters and error words exist once per parity of the epoch, and the workgroup that
draws ticket 0 zeroes the other parity's for the launch after it.  With 16-bit passed states an item's last state is
stored twice -- rounded into `out`, exact into a slot of the workspace that the next item reads instead of `out` -- and
those slots are never cleared: the last test keeps a workspace full of stale slots and checks that the final states are
those of the exact recurrence and `out` is that recurrence rounded once."""
import random

import pytest


class Workspace:
    """What survives from launch to launch when the caller keeps a workspace and passes epochs (ssd_fused_opts.epoch):
    two banks of ticket counters and two error words, by parity of the epoch; the epoch of the last launch; flags that
    hold the epoch they were raised in.  Cleared = all zero."""

    def __init__(self, n_flags=4096, cleared=None, garbage=0):
        self.tickets = [0, 0]
        self.errors = [0, 0]
        self.last_epoch = 0
        # a clearing covers the flags the call that asked for it looks at; what lies behind holds whatever the memory
        # held before (`garbage`)
        self.cleared = n_flags if cleared is None else cleared
        self.flags = [0] * self.cleared + [garbage] * (n_flags - self.cleared)
        self.carry = [float("nan")] * n_flags      # exact copies of the states that cross between items; never cleared

    def clear(self, n):
        """What a call with epoch 0 does first: zero for the n flags it looks at, and a record of n."""
        self.tickets, self.errors, self.last_epoch, self.cleared = [0, 0], [0, 0], 0, n
        self.flags[:n] = [0] * n

    def status(self):
        return self.errors[self.last_epoch & 1]


class _Flags:
    """One unit's row of flags inside the workspace: truthy = raised in the current epoch."""

    def __init__(self, ws, base, epoch):
        self.ws, self.base, self.epoch = ws, base, epoch

    def __getitem__(self, c):
        return self.ws.flags[self.base + c] == self.epoch

    def __setitem__(self, c, v):
        assert v == 1
        self.ws.flags[self.base + c] = self.epoch


class Launch:
    def __init__(self, n_units, C, R, n_wg, resident, spin_limit, seed, boundaries=(), ws=None, epoch=1, rounded=False):
        self.n_units, self.C, self.R, self.n_wg, self.resident, self.spin_limit = n_units, C, R, n_wg, resident, spin_limit
        self.rng = random.Random(seed)
        self.n_super = (C + R - 1) // R
        self.total = n_units * self.n_super
        self.ws = ws if ws is not None else Workspace()
        self.epoch, self.bank = epoch, epoch & 1
        assert n_units * (C + 1) <= len(self.ws.flags)
        self.flag = [_Flags(self.ws, u * (C + 1), epoch) for u in range(n_units)]
        # per (unit, chunk): chunk state S and decay d (zero where a sequence starts)
        self.S = [[self.rng.uniform(-1, 1) for _ in range(C)] for _ in range(n_units)]
        self.d = [[0.0 if (u, c) in boundaries else self.rng.uniform(0.1, 0.9) for c in range(C)] for u in range(n_units)]
        self.init = [self.rng.uniform(-1, 1) for _ in range(n_units)]
        self.out = [[None] * (C + 1) for _ in range(n_units)]       # out[u][c] = state entering chunk c; [C] = final
        self.events = 0
        # rounded: `out` holds rounded states (16-bit passed states), the exact ones cross through self.ws.carry
        self.rounded = rounded
        self.rnd = (lambda v: round(v, 2)) if rounded else (lambda v: v)

    def slot(self, u, c):
        return u * self.n_super + c // self.R

    @property
    def ticket(self):
        return self.ws.tickets[self.bank]

    @property
    def error(self):
        return self.ws.errors[self.bank]

    @error.setter
    def error(self, v):
        self.ws.errors[self.bank] = v

    def draw(self):
        t = self.ws.tickets[self.bank]
        self.ws.tickets[self.bank] += 1
        if t == 0:
            # is the workspace what the epoch promises?  The launch before was epoch - 1 (0 after a clearing), and the
            # flags this launch looks at were covered by the last clearing
            if self.ws.last_epoch != self.epoch - 1 or self.ws.cleared < self.n_units * (self.C + 1):
                self.error |= 4
            # one workgroup per launch: what the next epoch (the other parity) must find at zero
            self.ws.tickets[self.bank ^ 1] = 0
            self.ws.errors[self.bank ^ 1] = 0
            self.ws.last_epoch = self.epoch
        return t

    def item(self, t):
        k, u = divmod(t, self.n_units)
        return u, k * self.R, min(self.C, (k + 1) * self.R)

    def workgroup(self):
        """One persistent workgroup as a generator: every `yield` is a point where the scheduler may switch."""
        cur = self.draw()
        if cur >= self.total:
            # nothing to do -- or counters that a launch two epochs back left behind, in which case nobody draws
            # ticket 0 and this is where the broken promise shows
            if self.ws.last_epoch not in (self.epoch - 1, self.epoch):
                self.error |= 4
            return
        u, c0, c1 = self.item(cur)
        single = c1 - c0 == 1
        nxt = self.draw() if single else None          # a first item of one chunk needs its successor at once
        late = nxt is None
        after = None
        yield
        while cur < self.total:
            u, c0, c1 = self.item(cur)
            n = c1 - c0
            held = []
            for r in range(n):                         # the chunks of the item: independent of every other chunk
                if r == 0 or (late and r == 1):
                    t_new = self.draw()
                    if late and r == 0:
                        nxt = t_new
                    else:
                        after = t_new
                held.append(self.S[u][c0 + r])
                yield
            scale = [self.d[u][c0 + r] for r in range(n)]
            jz = max([r for r in range(1, n) if scale[r] == 0.0], default=0)

            def hand_on():
                if c0 + n < self.C:
                    if self.rounded:
                        self.ws.carry[self.slot(u, c0 + n)] = held[n - 1]
                    self.out[u][c0 + n] = self.rnd(held[n - 1])
                else:
                    self.out[u][c0 + n] = held[n - 1]  # the final state is never rounded
                yield                                  # the stores are acknowledged ...
                if c0 + n < self.C:
                    self.flag[u][c0 + n] = 1           # ... before the flag goes up

            if jz > 0:                                 # a sequence starts inside the item: the part behind it first
                for r in range(jz + 1, n):
                    held[r] += scale[r] * held[r - 1]
                yield from hand_on()
            use_prev = scale[0] != 0.0
            if use_prev and c0 > 0:
                polls = 0
                while not self.flag[u][c0]:
                    polls += 1
                    if polls >= self.spin_limit:
                        self.error |= 1
                        break
                    yield
            if c0 == 0:
                self.out[u][0] = self.rnd(self.init[u])
            if use_prev:
                if c0 == 0:
                    prev = self.init[u]
                elif self.rounded:
                    prev = self.ws.carry[self.slot(u, c0)]                                  # gave up: whatever is there
                else:
                    prev = self.out[u][c0] if self.out[u][c0] is not None else float("nan")
                held[0] += scale[0] * prev
            for r in range(1, jz if jz > 0 else n):
                held[r] += scale[r] * held[r - 1]
            if jz == 0:
                yield from hand_on()
            for r in range(n - 1):                     # the states inside the item
                self.out[u][c0 + r + 1] = self.rnd(held[r])
            yield
            cur, nxt, after, late = nxt, after, None, False

    def run(self):
        waiting = [self.workgroup() for _ in range(self.n_wg)]      # dispatched in order, `resident` at a time
        running = []
        budget = 200 * (self.total + self.n_wg) * max(4, min(self.spin_limit, 64))
        while waiting or running:
            while waiting and len(running) < self.resident:
                running.append(waiting.pop(0))
            g = self.rng.choice(running)
            try:
                next(g)
            except StopIteration:
                running.remove(g)
            self.events += 1
            assert self.events < budget, "the launch does not drain"
        return self

    def reference(self):
        want = []
        for u in range(self.n_units):
            s, row = self.init[u], [self.init[u]]
            for c in range(self.C):
                s = self.d[u][c] * s + self.S[u][c]
                row.append(s)
            want.append(row)
        return want


SHAPES = [(5, 32, 4, 32), (1, 16, 4, 8), (7, 9, 2, 16), (3, 5, 1, 8), (40, 8, 4, 16), (2, 1, 4, 4), (6, 3, 4, 64)]


@pytest.mark.parametrize("resident", [1, 2, 3, 1000])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "units%d-C%d-R%d-wg%d" % s)
def test_every_schedule_drains_and_matches_the_serial_recurrence(shape, resident):
    n_units, C, R, n_wg = shape
    for seed in range(12):
        rng = random.Random(1000 + seed)
        boundaries = {(rng.randrange(n_units), rng.randrange(C)) for _ in range((n_units * C) // 7)} if seed % 2 else set()
        L = Launch(n_units, C, R, n_wg, resident, spin_limit=1 << 30, seed=seed, boundaries=boundaries).run()
        assert L.error == 0
        assert L.ticket >= L.total
        want = L.reference()
        for u in range(n_units):
            for c in range(C + 1):
                assert L.out[u][c] is not None, (u, c)
                assert abs(L.out[u][c] - want[u][c]) <= 1e-12 * max(1.0, abs(want[u][c])), (u, c, seed)


def test_an_item_only_ever_waits_for_a_smaller_ticket():
    # the order argument itself: the item a ticket depends on has the ticket `units` below it
    L = Launch(5, 32, 4, 32, 1000, 1 << 30, 0)
    for t in range(L.total):
        u, c0, _ = L.item(t)
        if c0 > 0:
            up, _, c1p = L.item(t - L.n_units)
            assert up == u and c1p == c0


@pytest.mark.parametrize("resident", [2, 1000])
def test_a_wait_that_runs_out_is_reported_and_the_launch_still_drains(resident):
    reported = 0
    for seed in range(20):
        L = Launch(3, 16, 1, 16, resident, spin_limit=1, seed=seed).run()
        reported += L.error
        for u in range(3):
            assert not L.flag[u][16] and all(L.flag[u][c] for c in range(1, 16))     # every flag was raised all the same
    assert reported > 0
    # and with one resident workgroup nothing ever waits: it meets its own finished items
    assert Launch(3, 16, 1, 16, 1, spin_limit=1, seed=0).run().error == 0


def test_a_workspace_kept_from_launch_to_launch_with_epochs():
    # no clearing between launches: shapes, chunks per item and residency change, one launch has a wait that runs out;
    # every launch drains, computes the serial recurrence, and reports its own error word only
    rng = random.Random(5)
    ws = Workspace()
    epoch = 1
    for i in range(40):
        n_units, C, R, n_wg = rng.choice(SHAPES)
        limit = 1 if i % 9 == 4 else 1 << 30
        resident = rng.choice([1, 2, 3, 1000])
        boundaries = {(rng.randrange(n_units), rng.randrange(C)) for _ in range((n_units * C) // 7)} if i % 2 else set()
        L = Launch(n_units, C, R, n_wg, resident, spin_limit=limit, seed=100 + i, boundaries=boundaries, ws=ws, epoch=epoch).run()
        assert ws.last_epoch == epoch
        assert L.ticket >= L.total
        if limit > 1:
            assert ws.status() == 0, i
            want = L.reference()
            for u in range(n_units):
                for c in range(C + 1):
                    assert abs(L.out[u][c] - want[u][c]) <= 1e-12 * max(1.0, abs(want[u][c])), (i, u, c)
        epoch += 1
    assert ws.tickets[epoch & 1] == 0            # the bank of the launch that would come next is clean


def test_rounded_passed_states_cross_between_items_exactly():
    # 16-bit `out`: the state entering an item is read from the workspace slot its predecessor wrote in this launch,
    # never from the rounded `out` and never from what an earlier launch (other sizes, other slot mapping) left there
    rng = random.Random(11)
    ws = Workspace()
    epoch = 1
    for i in range(40):
        n_units, C, R, n_wg = rng.choice([sh for sh in SHAPES if sh[2] > 1])
        resident = rng.choice([1, 2, 3, 1000])
        boundaries = {(rng.randrange(n_units), rng.randrange(C)) for _ in range((n_units * C) // 7)} if i % 2 else set()
        L = Launch(n_units, C, R, n_wg, resident, spin_limit=1 << 30, seed=300 + i, boundaries=boundaries, ws=ws, epoch=epoch,
                   rounded=i % 3 != 2).run()
        assert ws.status() == 0, i
        want = L.reference()
        for u in range(n_units):
            assert abs(L.out[u][C] - want[u][C]) <= 1e-12 * max(1.0, abs(want[u][C])), (i, u)
            for c in range(C):
                assert abs(L.out[u][c] - L.rnd(want[u][c])) <= (1e-2 + 1e-9 if L.rounded else 1e-12 * max(1.0, abs(want[u][c]))), (i, u, c)
        epoch += 1


def test_flags_behind_the_cleared_part_are_not_trusted():
    """A kept workspace is cleared for the call that starts its epochs; a later call with more (unit, chunk) pairs looks
    at flags behind that part, which hold whatever the memory held -- here the very value of the coming epoch, so
    every wait would be skipped.  The kernel's check at ticket 0 reports it; the host policy of the wrappers (clear again
    when a call needs more flags than the last clearing covered) avoids it."""
    small, big = (3, 5, 1, 8), (7, 9, 2, 16)
    n_small, n_big = small[0] * (small[1] + 1), big[0] * (big[1] + 1)
    wrong = 0
    for seed in range(10):
        ws = Workspace(cleared=n_small, garbage=2)
        Launch(*small, 1000, spin_limit=1 << 30, seed=seed, ws=ws, epoch=1).run()
        assert ws.status() == 0
        L = Launch(*big, 1000, spin_limit=1 << 30, seed=50 + seed, ws=ws, epoch=2).run()
        assert ws.status() & 4                       # reported ...
        want = L.reference()
        wrong += any(L.out[u][c] is None or not abs(L.out[u][c] - want[u][c]) <= 1e-9 for u in range(big[0]) for c in range(big[1] + 1))
        # the host policy: this call needs more flags than were cleared -> epoch 0, i.e. clear, then launch as epoch 1
        ws = Workspace(cleared=n_small, garbage=2)
        Launch(*small, 1000, spin_limit=1 << 30, seed=seed, ws=ws, epoch=1).run()
        ws.clear(n_big)
        L = Launch(*big, 2, spin_limit=1 << 30, seed=50 + seed, ws=ws, epoch=1).run()
        assert ws.status() == 0
        want = L.reference()
        assert all(abs(L.out[u][c] - want[u][c]) <= 1e-12 * max(1.0, abs(want[u][c])) for u in range(big[0]) for c in range(big[1] + 1))
    assert wrong > 0                                 # ... and with reason: skipped waits do give wrong states
    # an epoch that does not follow the one before is reported as well
    ws = Workspace()
    Launch(*small, 1000, spin_limit=1 << 30, seed=0, ws=ws, epoch=1).run()
    Launch(*small, 1000, spin_limit=1 << 30, seed=1, ws=ws, epoch=3).run()
    assert ws.status() & 4
