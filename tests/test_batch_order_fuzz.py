"""Batches whose threads order one another by notifies, on random programs (recorder threads, no GPU).

A random, deadlock-free program is made by drawing a global sequence of events - thread t copies, thread a posts to
thread b, thread b waits for it, on a slot that only a posts to - and giving every thread its own events in that order; the calls are then made
thread by thread (so most waits are CALLED before the records that satisfy them), all inside one HcommBatchModeStart /
End pair.  With one segment per launch (HCOMM_GFX_MAX_SEGMENTS=1, read once per process: hence the child process) the
first thread's launch log is the order HcommBatchModeEnd settled on, every copy recognisable by its length.  Checked:
every copy appears exactly once; each thread's copies keep their order; a copy a thread makes after a wait comes after
every copy the posting thread made before the matching record; programs with one wait too many end in HCCL_E_TIMEOUT
with nothing issued and every thread usable again."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r'''
import random, sys
sys.path.insert(0, %(root)r)
import hcomm_amd as h
R = h.HcclResult
rng = random.Random(%(seed)d)
checked = 0
for trial in range(%(trials)d):
    nt = rng.randint(2, 9)
    th = [h.HcommGfxRecorderThreadAlloc()[1] for _ in range(nt)]
    events = []                      # the global order the program is consistent with
    per_thread = [[] for _ in range(nt)]
    pending = []                     # posts not yet waited for: (poster, waiter, slot)
    next_id = 1
    for _ in range(rng.randint(1, 120)):
        kind = rng.random()
        if kind < 0.5:
            t = rng.randrange(nt)
            per_thread[t].append(("copy", next_id)); events.append((t, "copy", next_id)); next_id += 1
        elif kind < 0.78 or not pending:
            a, b = rng.sample(range(nt), 2)
            slot = a + 9 * rng.randrange(3)   # a slot has ONE poster (as in the schedules: a slot per peer), so its records are met in the order issued
            per_thread[a].append(("post", b, slot)); pending.append((a, b, slot, len(events))); events.append((a, "post", b, slot))
        else:
            # the OLDEST pending post of some (waiter, slot): records of a slot are consumed in the order issued
            i = rng.randrange(len(pending))
            a, b, slot, at = pending[i]
            j = min(k for k, p in enumerate(pending) if p[1] == b and p[2] == slot)
            a, b, slot, at = pending.pop(j)
            per_thread[b].append(("wait", slot, a, at)); events.append((b, "wait", slot, a, at))
    dead = rng.random() < 0.25
    if dead:                         # a wait nothing will ever satisfy: a slot no post of the program is left on
        b = rng.randrange(nt)
        free = [s for s in range(32) if not any(p[1] == b and p[2] == s for p in pending)]
        per_thread[b].insert(rng.randint(0, len(per_thread[b])), ("wait", free[0], None, None))
    first = next((t for t in rng.sample(range(nt), nt) if per_thread[t]), 0)
    order = [first] + [t for t in range(nt) if t != first]
    assert h.HcommBatchModeStart(b"fuzz") == 0
    for t in order:
        for ev in per_thread[t]:
            if ev[0] == "copy":
                assert h.HcommLocalCopyOnThread(th[t], (1 << 40) + (ev[1] << 24), (1 << 41) + (ev[1] << 24), 16 * ev[1]) == 0
            elif ev[0] == "post":
                assert h.HcommThreadNotifyRecordOnThread(th[t], th[ev[1]], ev[2]) == 0
            else:
                assert h.HcommThreadNotifyWaitOnThread(th[t], ev[1], 5) == 0
    rc = h.HcommBatchModeEnd(b"fuzz")
    logs = [[l.bytes // 16 for l in h.launch_log(x)] for x in th]
    if dead:
        assert rc == R.E_TIMEOUT, (trial, rc)
        assert not any(logs), trial
        assert h.HcommLocalCopyOnThread(th[0], 1 << 40, 1 << 41, 16) == 0      # free again
    else:
        assert rc == 0, (trial, rc)
        if not any(ev[0] != "copy" for evs in per_thread for ev in evs):
            # no notify in the batch: every thread's copies go to its own stream, as in any batch
            for t in range(nt):
                assert logs[t] == [ev[1] for ev in per_thread[t]], (trial, "plain batch", t)
            h.HcommThreadFree(th)
            checked += 1
            continue
        got = logs[first]
        assert all(not l for i, l in enumerate(logs) if i != first), trial
        want_ids = [ev[1] for t in range(nt) for ev in per_thread[t] if ev[0] == "copy"]
        assert sorted(got) == sorted(want_ids), (trial, "every copy once")
        where = {c: i for i, c in enumerate(got)}
        for t in range(nt):
            mine = [where[ev[1]] for ev in per_thread[t] if ev[0] == "copy"]
            assert mine == sorted(mine), (trial, "thread order", t)
        for t in range(nt):
            for k, ev in enumerate(per_thread[t]):
                if ev[0] != "wait":
                    continue
                poster, at = ev[2], ev[3]
                before = [e[2] for e in events[:at] if e[0] == poster and e[1] == "copy"]
                after = [e[1] for e in per_thread[t][k + 1:] if e[0] == "copy"]
                if before and after:
                    assert max(where[c] for c in before) < min(where[c] for c in after), (trial, "record before wait", t, ev)
        # every record met its wait, or is still there for a later one
        left = sum(1 for p in pending)
        found = 0
        for b in range(nt):
            for s in range(32):
                while h.HcommThreadNotifyWaitOnThread(th[b], s, 0) == 0:
                    found += 1
        assert found == left, (trial, found, left)
    h.HcommThreadFree(th)
    checked += 1
print("checked", checked)
'''


def test_random_programs_of_copies_posts_and_waits_in_one_batch():
    env = dict(os.environ, HCOMM_GFX_MAX_SEGMENTS="1")
    for seed in (1, 2, 3, 4, 5, 6):
        run = subprocess.run([sys.executable, "-c", CHILD % {"root": ROOT, "seed": seed, "trials": 150}],
                             capture_output=True, text=True, timeout=600, env=env)
        assert run.returncode == 0, (seed, run.stdout[-500:], run.stderr[-3000:])
        assert "checked 150" in run.stdout
