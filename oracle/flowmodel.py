"""Explicit-state model of the staging flow control.  Test infrastructure,
never shipped.

What is modelled (the design in ``mintccl_amd/csrc/ring.hpp``): one
wave-channel of a pipeline with positions ``0..hops``.  Position ``h`` sends
step ``s`` as ``lines`` separate line writes into slot ``s % nslots`` of
position ``h + 1``; a line carries the flag ``s * lines + l + 1`` (unique over
the transfer, like the reference's line numbers, ``2_sendrecv_indirect.py:61``).
A receiver takes a line only when the slot shows exactly the flag it expects
(``recv_ll128``, ``protocol.py:111,126``).  After it has taken every line of
step ``s`` it publishes ``tail = s + 1``; a sender may write step ``s`` only if
``s - tail < nslots`` (the separate credit word that replaces
``wait_ll128`` / ``post_ll128``, ``protocol.py:161-189``).  Middle positions
forward line ``l`` of step ``s`` right after taking it.

``explore`` walks every interleaving of the positions' atomic actions (one
line write, one line poll, one credit write, one credit read) and reports

* ``overwritten`` - a slot line was overwritten before its reader had taken it,
* ``wrong``       - a reader accepted a payload that is not the one for the
                    line it expected,
* ``deadlocks``   - reachable non-final states with no enabled action
                    ("would spin forever"),
* ``finals``      - number of distinct final states (all lines delivered).

``post_early=True`` models the reference's defect (credit published at the
start of a round, before the slot has been drained - ``3_sendrecv_buffer.py:49-52``
with ``protocol.py:183-189``); ``drop=(h, s, l)`` loses one line write.  Both
must be caught, which is how the tests know the checker has teeth.

``explore_temporal`` does the same for the temporal allgather, where one agent
per position serves a different rank in every phase and the ranks' credit
words change hands (``mintccl_amd/csrc/temporal.hpp``).

Pinning: this is a model of the build's own protocol, checked by invariants
(no reference vectors exist for flow control).
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass


@dataclass
class Result:
    states: int = 0
    overwritten: int = 0
    wrong: int = 0
    deadlocks: int = 0
    finals: int = 0


def explore(hops: int, nslots: int, steps: int, lines: int = 1, post_early: bool = False,
            drop: tuple | None = None, max_states: int = 2_000_000) -> Result:
    npos = hops + 1
    nlines = steps * lines
    # per position: pc = number of line-actions completed (0..nlines), and a
    # phase inside the current line for middle positions (0 = must take,
    # 1 = must forward).  slot[h][i] = (flag, payload, taken) for receiver h.
    # tail[h] = credit published by receiver h; seen[h] = last credit value
    # sender h has read from receiver h + 1.
    empty_slots = tuple((0, 0, True) for _ in range(nslots * lines))
    init = (tuple(0 for _ in range(npos)),            # pc
            tuple(0 for _ in range(npos)),            # phase
            tuple(empty_slots for _ in range(npos)),  # slots (index 0 unused)
            tuple(0 for _ in range(npos)),            # tail
            tuple(0 for _ in range(npos)))            # seen
    res = Result()
    seen_states = {init}
    todo = deque([init])

    def flag_of(idx: int) -> int:
        return idx + 1

    while todo:
        st = todo.popleft()
        res.states += 1
        if res.states > max_states:
            raise RuntimeError("state space larger than max_states")
        pc, phase, slots, tail, seen = st
        succ = []
        for h in range(npos):
            idx = pc[h]
            if idx >= nlines:
                continue
            s, l = divmod(idx, lines)
            recv, send = h > 0, h < hops
            want_take = recv and phase[h] == 0
            if want_take:
                cell = slots[h][(s % nslots) * lines + l]
                if cell[0] == flag_of(idx) and not cell[2]:
                    ok = cell[1] == idx            # payload belongs to the line
                    sl = list(slots[h]); sl[(s % nslots) * lines + l] = (cell[0], cell[1], True)
                    ns = list(slots); ns[h] = tuple(sl)
                    npc, nph, nt = list(pc), list(phase), list(tail)
                    if send:
                        nph[h] = 1
                    else:
                        npc[h] = idx + 1
                        if l == lines - 1 and not post_early:
                            nt[h] = s + 1
                    succ.append(((tuple(npc), tuple(nph), tuple(ns), tuple(nt), seen), ok))
                continue
            # sending (origin, or a middle position in phase 1)
            need_credit = s >= nslots and seen[h] < s - nslots + 1
            if need_credit:
                if tail[h + 1] != seen[h]:
                    nseen = list(seen); nseen[h] = tail[h + 1]
                    succ.append(((pc, phase, slots, tail, tuple(nseen)), True))
                continue
            tgt = slots[h + 1]
            cell_i = (s % nslots) * lines + l
            over = not tgt[cell_i][2]
            if drop == (h, s, l):
                new_cell = tgt[cell_i]
                over = False
            else:
                new_cell = (flag_of(idx), idx, False)
            sl = list(tgt); sl[cell_i] = new_cell
            ns = list(slots); ns[h + 1] = tuple(sl)
            npc, nph, nt = list(pc), list(phase), list(tail)
            npc[h] = idx + 1
            nph[h] = 0
            if recv and l == lines - 1 and not post_early:
                nt[h] = s + 1                       # drained step s, then forwarded it
            succ.append(((tuple(npc), tuple(nph), tuple(ns), tuple(nt), seen),
                         "over" if over else True))
        if post_early:
            # defective credit: a receiver may publish "step s drained" as
            # soon as it *starts* step s (before taking its lines)
            for h in range(1, npos):
                idx = pc[h]
                if idx < nlines:
                    s = idx // lines
                    if tail[h] < s + 1 and phase[h] == 0 and idx % lines == 0:
                        nt = list(tail); nt[h] = s + 1
                        succ.append(((pc, phase, slots, tuple(nt), seen), True))
        if not succ:
            if all(p >= nlines for p in pc):
                res.finals += 1
            else:
                res.deadlocks += 1
            continue
        for nxt, verdict in succ:
            if verdict == "over":
                res.overwritten += 1
            elif verdict is False:
                res.wrong += 1
            if nxt not in seen_states:
                seen_states.add(nxt)
                todo.append(nxt)
    return res


def explore_temporal(world: int, nslots: int, steps: int, handover: bool = True,
                     max_states: int = 4_000_000) -> Result:
    """The temporal allgather (``mintccl_amd/csrc/temporal.hpp``): ``world``
    phases, phase c a broadcast of row c from rank c round the ring; one agent
    per *position* that serves, in phase c, the rank c + position.  Steps are
    numbered through the phases; a rank has ``nslots`` slots and one credit
    word, which a different agent posts in every phase.  ``handover`` is the
    rule that makes that safe: before its first post of a phase an agent waits
    until the word has reached the phase's first step (the origin, whose
    rank's slots stay empty, posts the whole phase at its end and waits
    there).  Without it an agent can publish a later count while the agent
    that served the rank before has not emptied its last slots - the checker
    must report that as ``overwritten`` (or as the deadlock a count that went
    backwards leads to)."""
    S = steps

    def need(gs: int) -> int:
        return max(0, gs - nslots + 1)

    programs = []
    for h in range(world):
        prog = []
        for c in range(world):
            rank, nxt, base = (c + h) % world, (c + h + 1) % world, c * S
            if h and handover and base:
                prog.append(("wait_tail", rank, base))
            for s in range(S):
                gs = base + s
                if h == 0:
                    prog += [("wait_tail", nxt, need(gs)), ("write", nxt, gs)]
                else:
                    prog += [("poll", rank, gs), ("post", rank, gs + 1)]
                    if h < world - 1:
                        prog += [("wait_tail", nxt, need(gs)), ("write", nxt, gs)]
            if h == 0:
                if handover and base:
                    prog.append(("wait_tail", rank, base))
                prog.append(("post", rank, base + S))
        programs.append(prog)

    # state: pc per agent; per rank the slots as (tag, taken); per rank the credit word
    init = (tuple(0 for _ in range(world)),
            tuple(tuple((0, True) for _ in range(nslots)) for _ in range(world)),
            tuple(0 for _ in range(world)))
    res = Result()
    seen_states = {init}
    todo = deque([init])
    while todo:
        st = todo.popleft()
        res.states += 1
        if res.states > max_states:
            raise RuntimeError("state space larger than max_states")
        pc, slots, tail = st
        succ = []
        for h in range(world):
            if pc[h] >= len(programs[h]):
                continue
            kind, r, x = programs[h][pc[h]]
            nslots_r, ntail, bad = slots, tail, None
            if kind == "wait_tail":
                if tail[r] < x:
                    continue
            elif kind == "poll":
                tag, taken = slots[r][x % nslots]
                if tag != x + 1:
                    continue
                if taken:
                    bad = "wrong"           # taken twice
                row = list(slots[r]); row[x % nslots] = (tag, True)
                nslots_r = slots[:r] + (tuple(row),) + slots[r + 1:]
            elif kind == "write":
                tag, taken = slots[r][x % nslots]
                if not taken:
                    bad = "over"
                row = list(slots[r]); row[x % nslots] = (x + 1, False)
                nslots_r = slots[:r] + (tuple(row),) + slots[r + 1:]
            else:                           # post: a plain store, it may also lower the word
                ntail = tail[:r] + (x,) + tail[r + 1:]
            npc = pc[:h] + (pc[h] + 1,) + pc[h + 1:]
            succ.append(((npc, nslots_r, ntail), bad))
        if not succ:
            if all(pc[h] >= len(programs[h]) for h in range(world)):
                res.finals += 1
            else:
                res.deadlocks += 1
            continue
        for nxt_state, bad in succ:
            if bad == "over":
                res.overwritten += 1
                continue
            if bad == "wrong":
                res.wrong += 1
                continue
            if nxt_state not in seen_states:
                seen_states.add(nxt_state)
                todo.append(nxt_state)
    return res
