"""The work-queue launch protocol, walked through on the CPU.

Two models, both exhaustive over every interleaving of a small launch:

* the counters in device memory (natten_amd/csrc/work_queue.hpp, compiled here with g++ so that the
  model runs the kernels' own decision functions): every launch position is handed out exactly once,
  every workgroup ends after at most `nq * per_queue + nq` increments, nobody touches a counter once
  the last workgroup out has begun to store zeros, and the block is all zero when the launch ends;
* the hand-over of a position from thread 0 to the other waves of its workgroup through the two LDS
  slots of fna_queue_loop (natten_amd/csrc/fna_fwd.hpp): every wave reads, for every tile, the value
  thread 0 wrote for that tile.  LDS stores are modelled as the hardware performs them: issued by the
  wave, performed at some later point unless the wave waits for its LDS operations (`s_waitcnt
  lgkmcnt(0)`), and a barrier by itself does not wait for them.  The kernels therefore enter every
  barrier through workgroup_sync(), which waits first; without that wait a wave released by the barrier
  can read the slot before thread 0's store has been performed and gets the position of two tiles
  earlier -- the fault the work-queue launch had on launch positions past the end of a problem, where
  the compiler had placed no wait between the store and the barrier.

Each model is also run on deliberately broken protocols (zeros stored by the first workgroup out, a
return to a retired queue, counters that do not start at zero; one slot instead of two, a barrier
without the wait), which it must reject.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def wq(tmp_path_factory):
    out = tmp_path_factory.mktemp("queue_model") / "libqueue_model.so"
    cmd = ["g++", "-O1", "-std=c++17", "-shared", "-fPIC", os.path.join(HERE, "queue_model.cpp"), "-o", str(out)]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout
    lib = ctypes.CDLL(str(out))
    lib.wq_position.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_int), ctypes.c_uint32, ctypes.c_int, ctypes.c_int]
    lib.wq_last_one_out.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
    lib.wq_max_increments.restype = ctypes.c_longlong
    return lib


class Violation(Exception):
    pass


# ---------------------------------------------------------------------------------------------
# Model 1: the counters.  A workgroup is a small state machine; each of its steps is one atomic
# operation on the shared block (an atomicAdd that returns the old value, or a plain store).
# ---------------------------------------------------------------------------------------------
TAKE, DONE, RESET, END = 0, 1, 2, 3


def explore_counters(lib, nq, per_queue, workgroups, start=None, last_out=None, position=None):
    """Walks every interleaving.  start: initial counter values (default zeros).  last_out /
    position: replacements for the library's decisions (the broken protocols)."""
    stride = lib.wq_stride()
    last_out = last_out or (lambda left, n: bool(lib.wq_last_one_out(left, n)))

    def lib_position(home, victim, ticket):
        v = ctypes.c_int(victim)
        pos = lib.wq_position(home, ctypes.byref(v), ticket, per_queue, nq)
        return pos, v.value

    position = position or lib_position
    bound = lib.wq_max_increments(per_queue, nq)
    total = nq * per_queue
    # state: (counters tuple, done word, handed-out bitmask, per workgroup (pc, victim, increments, reset index))
    init = (tuple(start or [0] * nq), 0, 0, tuple((TAKE, 0, 0, 0) for _ in range(workgroups)))
    seen = {init}
    stack = [init]
    terminals = 0
    while stack:
        counters, done, handed, wgs = stack.pop()
        # the last workgroup out is storing zeros, or has finished doing so
        resetting = any(pc == RESET or (pc == END and ridx > 0) for pc, _, _, ridx in wgs)
        live = [w for w, (pc, *_) in enumerate(wgs) if pc != END]
        if not live:
            terminals += 1
            if handed != (1 << total) - 1:
                raise Violation(f"positions handed out: {handed:b}, expected all {total}")
            if any(counters) or done:
                raise Violation(f"block not zero at exit: {counters} done={done}")
            continue
        for w in live:
            pc, victim, incs, ridx = wgs[w]
            home = w % nq
            c, d, h = list(counters), done, handed
            if pc == TAKE:
                if resetting:
                    raise Violation("a counter is incremented while the last workgroup out stores zeros")
                q = lib.wq_counter_word(home, victim, nq) // stride
                ticket = c[q]
                c[q] += 1
                incs += 1
                if incs > bound:
                    raise Violation(f"workgroup {w} made {incs} increments, bound {bound}")
                pos, victim = position(home, victim, ticket)
                if pos >= 0:
                    if not 0 <= pos < total:
                        raise Violation(f"position {pos} outside the launch")
                    if h >> pos & 1:
                        raise Violation(f"position {pos} handed out twice")
                    h |= 1 << pos
                elif victim == nq:
                    pc = DONE
            elif pc == DONE:
                if resetting:
                    raise Violation("the done word is incremented while the last workgroup out stores zeros")
                left = d
                d += 1
                if last_out(left, workgroups):
                    pc, ridx = RESET, 0
                else:
                    pc = END
            else:  # RESET: nq counter stores, then the done word
                if ridx < nq:
                    c[ridx] = 0
                    ridx += 1
                else:
                    d = 0
                    pc = END
            nxt = (tuple(c), d, h, wgs[:w] + ((pc, victim, incs, ridx),) + wgs[w + 1:])
            if nxt not in seen:
                seen.add(nxt)
                stack.append(nxt)
    return len(seen), terminals


def test_layout_constants(wq):
    nq, stride = wq.wq_num_xcd(), wq.wq_stride()
    assert wq.wq_words() == nq * stride and stride * 4 == 64  # one counter per 64-byte line
    assert 0 < wq.wq_done_word() < stride  # shares the first queue's line, not its counter
    words = {wq.wq_counter_word(h, v, nq) for h in range(nq) for v in range(nq)}
    assert words == {x * stride for x in range(nq)}
    for h in range(nq):  # a workgroup visits every queue once, its own first
        order = [wq.wq_counter_word(h, v, nq) // stride for v in range(nq)]
        assert order[0] == h and sorted(order) == list(range(nq))


@pytest.mark.parametrize("nq,per_queue,workgroups", [
    (1, 3, 3), (2, 1, 2), (2, 2, 3), (2, 3, 2), (3, 1, 3), (3, 2, 3), (2, 0, 2), (4, 1, 2), (2, 2, 4),
])
def test_every_interleaving_small(wq, nq, per_queue, workgroups):
    states, terminals = explore_counters(wq, nq, per_queue, workgroups)
    assert terminals >= 1 and states > 0


def test_every_interleaving_eight_queues(wq):
    # the shipped queue count, two resident workgroups (homes 0 and 1) and three
    explore_counters(wq, wq.wq_num_xcd(), 1, 2)
    explore_counters(wq, wq.wq_num_xcd(), 2, 2)
    explore_counters(wq, wq.wq_num_xcd(), 1, 3)


def test_more_workgroups_than_positions(wq):
    explore_counters(wq, 2, 1, 4)


def test_model_rejects_reset_by_first_out(wq):
    # zeros stored by the first workgroup to leave instead of the last: others still increment
    with pytest.raises(Violation):
        explore_counters(wq, 2, 2, 3, last_out=lambda left, n: left == 0)


def test_model_rejects_returning_to_a_retired_queue(wq):
    # a workgroup that does not move on from an empty queue never ends: the increment bound catches it
    def stuck(home, victim, ticket):
        return (int(ticket) * 2 + (home + victim) % 2, victim) if ticket < 1 else (-1, victim)

    with pytest.raises(Violation):
        explore_counters(wq, 2, 1, 2, position=stuck)


def test_model_rejects_counters_that_do_not_start_at_zero(wq):
    # what `run_persistent = 2` asks its caller to vouch for: a stale count skips positions
    with pytest.raises(Violation):
        explore_counters(wq, 2, 2, 2, start=[1, 0])


# ---------------------------------------------------------------------------------------------
# Model 2: the hand-over inside a workgroup.  Every wave runs the loop of fna_queue_loop:
#   barrier; read s_pos[i]; leave if it is negative; the tile (some barriers; thread 0, in wave 0,
#   writes s_pos[i ^ 1] after the last of them -- a tile that returns at once has none);  i ^= 1.
# A step is a barrier arrival, an LDS read, the issue of an LDS write, or the LDS unit performing
# the oldest write a wave has issued: a write is not visible to the other waves before that, and
# only a wait for the wave's own LDS operations (what workgroup_sync() puts in front of every
# barrier) holds the wave until it has happened.  A barrier releases when every wave has arrived.
# Waves are otherwise free to run at any relative speed.
# ---------------------------------------------------------------------------------------------
def wave_program(wave, tiles, barriers_per_tile, write_at, wait_before_barrier):
    bar = [("wait",), ("bar",)] if wait_before_barrier else [("bar",)]
    ops = [("write", 0)] if wave == 0 else []
    for n, pid in enumerate(tiles):
        ops += bar + [("read", n)]
        if pid < 0:
            break
        if wave == 0 and write_at == "top":
            ops.append(("write", n + 1))
        ops += bar * barriers_per_tile[n % len(barriers_per_tile)]
        if wave == 0 and write_at == "end":
            ops.append(("write", n + 1))
    return ops


def explore_handover(waves, tiles, slots=2, barriers_per_tile=(2, 0, 1), write_at="end", wait_before_barrier=True):
    """tiles: the positions thread 0 obtains, in order, ending with a negative one."""
    progs = [wave_program(w, tiles, barriers_per_tile, write_at, wait_before_barrier) for w in range(waves)]
    # state: LDS slots, program counters, waves waiting at the barrier, writes issued by wave 0 and not yet performed
    init = ((None,) * slots, (0,) * waves, frozenset(), ())
    seen = {init}
    stack = [init]
    while stack:
        lds, pcs, waiting, pending = stack.pop()
        succ = []
        if pending:  # the LDS unit performs wave 0's oldest outstanding write
            l = list(lds)
            l[pending[0] % slots] = tiles[pending[0]]
            succ.append((tuple(l), pcs, waiting, pending[1:]))
        runnable = [w for w in range(waves) if pcs[w] < len(progs[w]) and w not in waiting]
        for w in runnable:
            op = progs[w][pcs[w]]
            pc, wt, pend = list(pcs), set(waiting), pending
            if op[0] == "wait":
                if w == 0 and pending:
                    continue  # held until its writes have been performed
                pc[w] += 1
            elif op[0] == "bar":
                wt.add(w)
                if len(wt) == sum(1 for x in range(waves) if pcs[x] < len(progs[x])):
                    for x in wt:
                        pc[x] += 1
                    wt = set()
            elif op[0] == "read":
                n = op[1]
                got = lds[n % slots]
                if w == 0:  # a wave sees its own writes in program order
                    for m in pending:
                        if m % slots == n % slots:
                            got = tiles[m]
                if got != tiles[n]:
                    raise Violation(f"wave {w} read {got} for its tile {n}; thread 0 wrote {tiles[n]} for it")
                pc[w] += 1
            else:
                pend = pending + (op[1],)
                pc[w] += 1
            succ.append((lds, tuple(pc), frozenset(wt), pend))
        if not succ:
            if waiting:
                raise Violation("deadlock: some waves wait at a barrier the others never reach")
            continue
        for nxt in succ:
            if nxt not in seen:
                seen.add(nxt)
                stack.append(nxt)
    return len(seen)


TILES = [5, 9, 2, 7, -1]


@pytest.mark.parametrize("waves", [2, 4])
@pytest.mark.parametrize("barriers", [(2,), (0,), (2, 0, 1), (0, 3)])
def test_handover_two_slots(waves, barriers):
    # the shipped form: thread 0 stores the next position after the tile's last barrier
    assert explore_handover(waves, TILES, slots=2, barriers_per_tile=barriers, write_at="end") > 0
    # ... and the form that stores it right after reading the current one
    assert explore_handover(waves, TILES, slots=2, barriers_per_tile=barriers, write_at="top") > 0


def test_handover_single_tile_and_empty_queue():
    explore_handover(4, [-1])
    explore_handover(4, [3, -1])


@pytest.mark.parametrize("write_at", ["end", "top"])
def test_model_rejects_one_slot(write_at):
    # with a single slot thread 0 may overwrite a position a slower wave has not read yet
    with pytest.raises(Violation):
        explore_handover(2, TILES, slots=1, barriers_per_tile=(0,), write_at=write_at)


@pytest.mark.parametrize("barriers", [(0,), (2, 0, 1)])
def test_model_rejects_a_barrier_without_the_wait_for_the_store(barriers):
    # The fault the work-queue launch had: on the path of a tile that returns at once nothing held
    # thread 0's wave between its store of the next position and the barrier at the top of the loop,
    # so another wave could read the slot before the store had been performed and work on the
    # position it held two tiles earlier.
    with pytest.raises(Violation):
        explore_handover(2, TILES, slots=2, barriers_per_tile=barriers, write_at="end", wait_before_barrier=False)
