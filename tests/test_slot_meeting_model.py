"""A model of how the chip places the workgroups of K-sliced GEMV launches, replayed on the CPU: does the fixed waiter of
the slot meeting (elutq_amd/csrc/hlq_gemv_dev.h: slices_meet_slots -- the workgroup of a column block's last K slice
polls the slots of the others) always get what it waits for, whatever else shares the GPU?

Model (what is assumed of the dispatcher, which no document promises -- hence the bounded wait in the kernel): the
workgroups of a launch go to the eight XCDs round robin by linear index (slice fastest, then column block); every XCD
places the workgroups it was given in index order, launch by launch, as places come free; an XCD has a fixed number
of places shared by all launches; which launch an XCD serves next is arbitrary (drawn at random here).  A worker (any
slice but the last) finishes once placed; the waiter finishes once placed AND all workers of its column block have
finished.  A run deadlocks when nothing can be placed and nothing can finish.

With 2, 4 or 8 slices waiters sit on XCDs 1, 3, 5, 7 only and wait for lower-numbered XCDs, so no run can deadlock;
with 3 slices waiters and the workers they wait for share XCDs and two oversubscribing launches can block each other --
which is why the launcher uses slots for 2, 4 or 8 slices only and arrival counters (nothing waits) otherwise."""
import random

XCDS = 8


def replay(launches, places, rng):
    """launches: list of (ksplit, ncb).  Returns True if every workgroup finishes."""
    queues = []                                # per launch, per XCD: workgroup indices in order
    for ks, ncb in launches:
        q = [[] for _ in range(XCDS)]
        for i in range(ks * ncb):
            q[i % XCDS].append(i)
        queues.append(q)
    placed = [[] for _ in range(XCDS)]         # (launch, index) of waiters that hold a place
    free = [places] * XCDS
    done_workers = [dict() for _ in launches]  # column block -> workers finished
    remaining = sum(ks * ncb for ks, ncb in launches)
    while remaining:
        progress = False
        for x in rng.sample(range(XCDS), XCDS):
            # waiters on this XCD whose workers are all done leave
            for item in list(placed[x]):
                li, i = item
                ks = launches[li][0]
                if done_workers[li].get(i // ks, 0) == ks - 1:
                    placed[x].remove(item)
                    free[x] += 1
                    remaining -= 1
                    progress = True
            # place workgroups while places are free, launches in random order, each launch in index order
            while free[x]:
                cands = [li for li in range(len(launches)) if queues[li][x]]
                if not cands:
                    break
                li = rng.choice(cands)
                i = queues[li][x].pop(0)
                ks = launches[li][0]
                progress = True
                if i % ks == ks - 1 and ks > 1:          # the waiter: holds its place until its workers are done
                    placed[x].append((li, i))
                    free[x] -= 1
                else:                                    # a worker finishes at once (its place is free again)
                    done_workers[li][i // ks] = done_workers[li].get(i // ks, 0) + 1
                    remaining -= 1
        if not progress:
            return False
    return True


def test_two_four_and_eight_slices_cannot_deadlock():
    rng = random.Random(1)
    for trial in range(300):
        n = rng.randint(1, 4)
        launches = [(rng.choice([2, 4, 8]), rng.randint(1, 80)) for _ in range(n)]
        places = rng.randint(1, 3)
        assert replay(launches, places, rng), (launches, places)


def test_three_slices_can_deadlock_when_launches_oversubscribe():
    """Two launches of three slices with one place per XCD: some placement order leaves every place held by a waiter
    whose workers are still queued behind another waiter."""
    rng = random.Random(2)
    stuck = sum(not replay([(3, 40), (3, 40)], 1, rng) for _ in range(200))
    assert stuck > 0
    # ... and a single launch cannot: its waiters are always behind their workers in every XCD's queue
    assert all(replay([(3, 64)], 1, rng) for _ in range(50))
