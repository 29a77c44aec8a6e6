"""A host-side model of the exchange that the long-row cross entropy kernel (seraph_amd/csrc/cross_entropy.hip,
ce_coop_kernel) runs between the P workgroups that share a row, stepped under adversarial schedules.

The kernel cannot be starved on purpose on a GPU, so the protocol is restated here as small coroutines (one per
workgroup, a scheduling point before every access to shared memory) and driven by schedulers that do what a busy
device may do: keep only a few workgroups resident at a time, let one run many rounds ahead of a partner that has
not started, give up on every wait at once.  The model has the kernel's moves in the kernel's order:

  load own part -> (max, sum) -> publish record[unit] (tag = launch, round) -> poll the partners' records a bounded
  number of times -> for a partner still missing: form its statistics from its logits in two sweeps, then look at its
  record once more and prefer that -> combine in part order -> overwrite the own part with the gradient (in place).

What must hold under every schedule: all partners of a row end up with the same (max, total), and it is the one the
row's original logits give.  The record layout of an earlier form of the kernel (two records per workgroup, chosen
by round parity) is modelled too and must FAIL under the same schedules: that is what shows the schedules bite."""
import math
import random

import pytest


def stats(vals):
    m = max(vals)
    s = 0.0
    for x in vals:
        s += math.exp(x - m)
    return (m, s)


def combine(parts):
    m, s = parts[0]
    for pm, ps in parts[1:]:
        nm = max(m, pm)
        s = s * math.exp(m - nm) + ps * math.exp(pm - nm)
        m = nm
    return (m, s)


class Device:
    def __init__(self, rows, P, G, width, per_unit_records, spin_limit, launch, seed):
        r = random.Random(seed)
        self.rows, self.P, self.G, self.width = rows, P, G, width
        self.logits = [[[r.gauss(0.0, 2.0) for _ in range(width)] for _ in range(P)] for _ in range(rows)]
        self.truth = [combine([stats(part) for part in row]) for row in self.logits]
        self.per_unit = per_unit_records
        self.records = {}                       # slot -> (tag, (m, s)); a slot holds one record, a store replaces it
        self.spin_limit = spin_limit
        self.launch = launch
        self.result = {}                        # unit -> (m, total) the workgroup used for its gradient
        self.fallbacks = 0

    def slot(self, g, round_, unit):
        return ("unit", unit) if self.per_unit else ("wg", round_ & 1, g)

    def workgroup(self, g):
        """Generator: yields before every access to shared memory (records, other parts' logits, own stores)."""
        P, G = self.P, self.G
        part, base = g % P, g - g % P
        round_ = 0
        u = g
        while u < self.rows * P:
            row = u // P
            yield
            mine = stats(list(self.logits[row][part]))                           # own part -> registers
            tag = (self.launch, round_)
            yield
            self.records[self.slot(g, round_, u)] = (tag, mine)                  # publish before any store
            parts = [None] * P
            for p in range(P):
                slot = self.slot(base + p, round_, row * P + p)
                for _ in range(self.spin_limit + 1):
                    yield
                    rec = self.records.get(slot)
                    if rec is not None and rec[0] == tag:
                        parts[p] = rec[1]
                        break
            for p in range(P):
                if parts[p] is not None:
                    continue
                self.fallbacks += 1
                seen = []
                for i in range(self.width):                                      # sweep 1 (maximum)
                    yield
                    seen.append(self.logits[row][p][i])
                m = max(seen)
                s = 0.0
                for i in range(self.width):                                      # sweep 2 (sum), re-reading memory
                    yield
                    s += math.exp(min(self.logits[row][p][i] - m, 50.0))
                yield
                rec = self.records.get(self.slot(base + p, round_, row * P + p))  # the record, once more
                parts[p] = rec[1] if rec is not None and rec[0] == tag else (m, s)
            total = combine(parts)
            self.result[u] = total
            for i in range(self.width):                                          # the gradient over the own logits
                yield
                self.logits[row][part][i] = 1e30 + i                              # anything but the logit
            u += G
            round_ += 1


def run(dev, schedule_seed, resident):
    """Runs all workgroups; at most `resident` are on the device at a time, admitted in index order as others finish
    (a workgroup that is not resident does not move).  Among residents the next to move is drawn at random, with a
    bias that lets some run far ahead."""
    r = random.Random(schedule_seed)
    waiting = [(g, dev.workgroup(g)) for g in range(dev.G)]
    r.shuffle(waiting) if schedule_seed % 3 == 0 else None                      # admission order is not the kernel's to choose
    live = []
    while waiting or live:
        while waiting and len(live) < resident:
            live.append(waiting.pop(0))
        k = 0 if r.random() < 0.6 else r.randrange(len(live))                    # favour one workgroup: it runs ahead
        try:
            next(live[k][1])
        except StopIteration:
            live.pop(k)


def all_agree(dev):
    ok = True
    for u, (m, s) in dev.result.items():
        tm, ts = dev.truth[u // dev.P]
        ok = ok and m == tm and abs(s - ts) <= 1e-12 * ts
    return ok and len(dev.result) == dev.rows * dev.P


CONFIGS = [  # rows, P, G, resident, spin_limit
    (12, 3, 6, 2, 0),
    (12, 3, 6, 4, 2),
    (20, 5, 5, 1, 0),          # one workgroup at a time: every wait fails, every partner's part is formed by hand
    (20, 5, 10, 3, 1),
    (9, 2, 4, 2, 0),
    (16, 4, 8, 8, 3),          # everybody resident: the ordinary case
]


@pytest.mark.parametrize("cfg", CONFIGS)
def test_every_partner_derives_the_rows_statistics_under_starving_schedules(cfg):
    rows, P, G, resident, spin = cfg
    fallbacks = 0
    for seed in range(40):
        dev = Device(rows, P, G, width=3, per_unit_records=True, spin_limit=spin, launch=7, seed=seed)
        run(dev, seed, resident)
        assert all_agree(dev), (cfg, seed)
        fallbacks += dev.fallbacks
    if resident < G:
        assert fallbacks > 0                                                     # the schedules did force the give-up path


def test_records_chosen_by_round_parity_fail_under_the_same_schedules():
    """The layout this kernel had before (record = [round & 1][workgroup]): a workgroup that gave up on a partner runs two
    rounds ahead, overwrites the record of the round its partner has yet to start, and its logits are gone too."""
    broken = 0
    for cfg in CONFIGS:
        rows, P, G, resident, spin = cfg
        for seed in range(40):
            dev = Device(rows, P, G, width=3, per_unit_records=False, spin_limit=spin, launch=7, seed=seed)
            run(dev, seed, resident)
            broken += not all_agree(dev)
    assert broken > 0


def test_a_record_left_by_another_launch_is_never_taken():
    dev = Device(6, 3, 3, width=3, per_unit_records=True, spin_limit=0, launch=8, seed=1)
    for u in range(18):
        dev.records[("unit", u)] = ((7, u // 3), (123.0, 1.0))                  # an older launch's records in the same slots
    run(dev, 5, 1)
    assert all_agree(dev)
