"""Host-side model of the loader / consumer protocol of the two ring kernels (the ring form of the Q4_K decode row
kernel, mh_matvec_rows.hip, and the row-owning small-batch kernel, mh_mmq_rows.hip), stepped under adversarial
schedules for every plan the library's own planners return over a grid of shapes. No GPU is involved: the plans come
from marmot_hip_rows_plan_probe, the state machines below restate what a loader and a consumer wavefront do with the
LDS counters.

The protocol: tasks (row segments) have a global order gi = 0, 1, ...; task gi lands in ring slot gi % nslots. Loader l
of L requests tasks l, l + L, ... with direct-to-LDS loads that complete in issue order, and publishes "task gi has
landed" (landed[slot] = gi + 1) from its outstanding-load count alone: behind the `outstanding` youngest instructions
everything has landed, and a task is taken to be ceil(outstanding / ipt) tasks back. Before it refills a slot it waits
for consumed[slot]; it keeps at most `lag` tasks in flight. A consumer takes its tasks in order, waits for landed and
releases the slot (consumed[slot] = gi + 1).

Checked for every plan, on a full workgroup and on the ragged last one:
  * safety: a task is never published while one of its load instructions is outstanding (this needs the per-task
    instruction count a loader divides by to be the number it really issues: with the slot size instead, rows whose
    last K segment is shorter published one instruction early), the 6-bit load counter never saturates, the tasks
    requested before the workgroup barrier fit the ring;
  * liveness: under eager, lazy (a load lands only when nobody can move) and random landing every consumer finishes.
    With the publishing rule the kernels first had (a loader that waits for a slot publishes nothing) the lazy
    schedule deadlocks on some plans: a consumer waits for a task of loader A, which waits for a slot whose consumer
    waits for a landed but unpublished task of loader B, which waits for a slot of the first consumer.
"""
import ctypes as C
import random

import pytest

Q4_K_BYTES = 144


class Unsafe(AssertionError):
    pass


class Deadlock(AssertionError):
    pass


def probe(lib, kernel, cus, N, K, M, nw, packed=0):
    out = (C.c_uint32 * 24)()
    st = lib.marmot_hip_rows_plan_probe(kernel, cus, N, K, M, nw, packed, out, 24)
    return list(out) if st == 0 else None


# ---------------------------------------------------------------- the two kernels as task lists
def matvec_rows_tasks(plan, K, rows_here, ipt_rule):
    """Per loader: [(gi, instructions issued)], the instruction count it divides by; per consumer: [gi]."""
    G, W, rows_per_wg, segs, seg_blocks, rpt, lag, pre, C_, nslots, slot_stride, grid, lds = plan[:13]
    nb = K // 256
    row_bytes = nb * Q4_K_BYTES
    L = W - C_
    assert L % segs == 0 and C_ % L == 0 and C_ % segs == 0  # what the loader loop's constant strides rely on
    groups = -(-rows_here // rpt)
    wstep, rg_step = C_ // segs, L // segs
    by_gi = {}
    consumers = []
    for c in range(C_):
        seg, wq = c % segs, c // segs
        mine = []
        rnd = 0
        rg = wq
        while rg < groups:
            gi = rnd * C_ + c
            by_gi[gi] = (rg, seg)
            mine.append(gi)
            rg += wstep
            rnd += 1
        consumers.append(mine)
    loaders, ipts = [], []
    for l in range(L):
        lseg, rg = l % segs, l // segs
        seg_first = lseg * seg_blocks
        seg_nb = min(nb - seg_first, seg_blocks)
        task_bytes = rpt * row_bytes if segs == 1 else seg_nb * Q4_K_BYTES
        issued_per_task = -(-task_bytes // 1024)  # whole KiBs and the partial one
        ipts.append(issued_per_task if ipt_rule == "issued" else slot_stride >> 10)
        mine = []
        gi = l
        while rg < groups:
            assert by_gi.get(gi) == (rg, lseg), f"loader {l} and the consumers disagree about task {gi}"
            mine.append((gi, issued_per_task))
            rg += rg_step
            gi += L
        loaders.append(mine)
    assert sorted(g for m in loaders for g, _ in m) == sorted(by_gi), "loaders and consumers cover different tasks"
    return dict(loaders=loaders, ipt=ipts, consumers=consumers, nslots=nslots, lag=lag, pre=pre, lag_prologue=None)


def mmq_rows_tasks(plan, ipt_rule):
    (NT, W, rows_per_wg, R, seg_blocks, segs, ks, spk, rgs_per_round, rounds, TC, C_, nslots, slot_stride, ipt, lag, pre,
     grid, lag_prologue, lds) = plan[:20]
    L = W - C_
    steps = rounds * spk
    issued_per_task = -(-(R * seg_blocks * Q4_K_BYTES) // 1024)  # the loader issues `ipt` instructions for every task
    assert issued_per_task == ipt
    loaders = [[(gi, ipt) for gi in range(l, steps * TC, L)] for l in range(L)]
    consumers = [[step * TC + c for step in range(steps)] for c in range(TC)]
    acc = ipt if ipt_rule == "issued" else slot_stride >> 10
    return dict(loaders=loaders, ipt=[acc] * L, consumers=consumers, nslots=nslots, lag=lag, pre=pre,
                lag_prologue=lag_prologue)


# ---------------------------------------------------------------- the protocol
def simulate(t, schedule, publish_while_waiting=True, seed=0):
    rng = random.Random(seed)
    nslots, lag, pre = t["nslots"], t["lag"], t["pre"]
    L = len(t["loaders"])
    landed = [0] * nslots
    consumed = [0] * nslots
    quantized = t["lag_prologue"] is None  # the decode kernel's loaders do not look at the quantization
    assert pre * L <= nslots and pre <= lag, "tasks requested before the barrier must not reuse a slot"

    class Loader:
        def __init__(self, l):
            self.l, self.todo, self.ipt = l, t["loaders"][l], t["ipt"][l]
            self.idx = self.issued = self.published = 0
            self.flight = []  # [gi, instructions outstanding], oldest first
            self.phase = "pre"
            self.max_out = 0

        def outstanding(self):
            return sum(n for _, n in self.flight)

        def land_one(self):
            for f in self.flight:
                if f[1] > 0:
                    f[1] -= 1
                    return True
            return False

        def issue(self):
            gi, n = self.todo[self.idx]
            self.flight.append([gi, n])
            self.idx += 1
            self.issued += 1
            self.max_out = max(self.max_out, self.outstanding())

        def publish(self):
            gi, left = self.flight.pop(0)
            if left != 0:
                raise Unsafe(f"loader {self.l} publishes task {gi} with {left} instructions outstanding")
            assert gi == self.todo[self.published][0]
            landed[gi % nslots] = gi + 1
            self.published += 1

        def publish_landed(self):
            pending = -(-self.outstanding() // self.ipt)
            moved = False
            while self.published + pending < self.issued:
                self.publish()
                moved = True
            return moved

        def wait_vmcnt_then_publish(self, allowed_tasks):
            """s_waitcnt vmcnt(allowed_tasks * ipt), then publish one task; False while it has to wait."""
            if self.outstanding() > allowed_tasks * self.ipt:
                return False
            self.publish()
            return True

        def run(self, barrier_open):
            moved = False
            while True:
                if self.phase == "pre":
                    while self.idx < min(pre, len(self.todo)):
                        self.issue()
                    self.phase = "barrier"
                    moved = True
                elif self.phase == "barrier":
                    if not barrier_open:
                        return moved
                    self.phase = "main"
                    moved = True
                elif self.phase == "main":
                    if self.idx == len(self.todo):
                        self.phase = "drain"
                        continue
                    if t["lag_prologue"] is not None and not quantized and self.issued - self.published >= t["lag_prologue"]:
                        if not self.wait_vmcnt_then_publish(t["lag_prologue"] - 1):
                            return moved
                        moved = True
                        continue
                    gi = self.todo[self.idx][0]
                    if gi >= nslots and consumed[gi % nslots] < gi - nslots + 1:
                        if publish_while_waiting and self.publish_landed():
                            moved = True
                        return moved  # spins
                    self.issue()
                    self.publish_landed()
                    moved = True
                    if self.issued - self.published >= lag:
                        self.phase = "lag"
                elif self.phase == "lag":
                    if not self.wait_vmcnt_then_publish(lag - 1):
                        return moved
                    self.phase = "main"
                    moved = True
                elif self.phase == "drain":
                    if self.published == self.issued:
                        self.phase = "done"
                        return True
                    if not self.wait_vmcnt_then_publish(self.issued - self.published - 1):
                        return moved
                    moved = True
                else:
                    return moved

    loaders = [Loader(l) for l in range(L)]
    cons_idx = [0] * len(t["consumers"])

    def run_consumers():
        moved = False
        if not quantized:
            return False
        order = list(range(len(cons_idx)))
        if schedule == "random":
            rng.shuffle(order)
        for c in order:
            todo = t["consumers"][c]
            while cons_idx[c] < len(todo):
                gi = todo[cons_idx[c]]
                if landed[gi % nslots] < gi + 1:
                    break
                assert landed[gi % nslots] == gi + 1, "a slot was refilled before its task was read"
                consumed[gi % nslots] = gi + 1
                cons_idx[c] += 1
                moved = True
                if schedule == "random" and rng.random() < 0.5:
                    break
        return moved

    barrier_open = False
    for _ in range(10_000_000):
        moved = False
        order = list(range(L))
        if schedule == "random":
            rng.shuffle(order)
        for l in order:
            moved |= loaders[l].run(barrier_open)
        if not barrier_open and all(ld.phase != "pre" for ld in loaders):
            barrier_open = True  # the consumers reach the barrier without waiting for anybody
            moved = True
        moved |= run_consumers()
        if all(ld.phase == "done" for ld in loaders) and all(i == len(td) for i, td in zip(cons_idx, t["consumers"])):
            assert all(ld.max_out <= 63 for ld in loaders), "the load counter holds six bits"
            return
        flying = [ld for ld in loaders if ld.outstanding() > 0]
        if schedule == "eager" or (schedule == "random" and rng.random() < 0.5):
            for ld in flying:
                while ld.land_one():
                    moved = True
        if moved:
            continue
        # nobody can move: the adversary has to give something
        if flying:
            (rng.choice(flying) if schedule == "random" else flying[0]).land_one()
        elif not quantized:
            quantized = True
        else:
            stuck = {c: t["consumers"][c][i] for c, i in enumerate(cons_idx) if i < len(t["consumers"][c])}
            raise Deadlock(f"nothing in flight, consumers wait for tasks {stuck}, loaders in "
                           f"{[(ld.phase, ld.idx, ld.published) for ld in loaders]}")
    raise AssertionError("the model did not terminate")


# ---------------------------------------------------------------- the plan space
CUS = 256
KS = [256, 512, 768, 1024, 2048, 2816, 3072, 4096, 5120, 8192, 11008, 13824, 14336, 16384, 28672]
MS = [64, 100, 1000, 1024, 4096, 4100, 11008, 14336, 32000, 128256]


def all_task_sets(lib, ipt_rule="issued"):
    for K in KS:
        for M in MS:
            for nw in (1, 2, 3):
                for N in (1, 2):
                    plan = probe(lib, 0, CUS, N, K, M, nw)
                    if plan is not None:
                        rows = plan[2]
                        for rows_here in {rows, M - (plan[11] - 1) * rows}:
                            yield f"decode N={N} {M}x{K} x{nw} rows={rows_here}", matvec_rows_tasks(plan, K, rows_here, ipt_rule)
                for N in (1, 3, 4, 5, 8, 9, 16):
                    for packed in (0, 1):
                        plan = probe(lib, 1, CUS, N, K, M, nw, packed)
                        if plan is not None:
                            yield f"small batch N={N} {M}x{K} x{nw} packed={packed}", mmq_rows_tasks(plan, ipt_rule)


@pytest.fixture(scope="module")
def lib():
    from marmot_amd import capi

    return capi.load_library()


def test_every_plan_is_safe_and_live(lib):
    n = reuse = 0
    for what, tasks in all_task_sets(lib):
        n += 1
        reuse += tasks["nslots"] < sum(len(m) for m in tasks["loaders"])
        for schedule, seeds in (("eager", (0,)), ("lazy", (0,)), ("random", (1, 2, 3))):
            for seed in seeds:
                try:
                    simulate(tasks, schedule, seed=seed)
                except (Unsafe, Deadlock) as e:
                    raise AssertionError(f"{what}, {schedule} landing, seed {seed}: {e}") from e
    assert n >= 300 and reuse >= 50, (n, reuse)  # the grid reaches plans whose ring is reused


def test_the_model_sees_the_two_defects_the_kernels_had(lib):
    """A loader that publishes nothing while it waits for a slot deadlocks under lazy landing on some plans; a loader
    that divides its outstanding instructions by the slot size instead of the number it issues per task publishes
    early where a row's last K segment is shorter (4096 x 11008: 43 blocks = 22 + 21)."""
    deadlocks = 0
    for what, tasks in all_task_sets(lib):
        try:
            simulate(tasks, "lazy", publish_while_waiting=False)
        except Deadlock:
            deadlocks += 1
    assert deadlocks > 0
    early = 0
    for what, tasks in all_task_sets(lib, ipt_rule="slot"):
        try:
            for schedule in ("eager", "lazy", "random"):
                simulate(tasks, schedule, seed=5)
        except Unsafe:
            early += 1
    assert early > 0
    plan = probe(lib, 0, CUS, 2, 11008, 4096, 1)
    assert plan is not None
    with pytest.raises(Unsafe):
        for seed in range(20):
            simulate(matvec_rows_tasks(plan, 11008, plan[2], "slot"), "random", seed=seed)
