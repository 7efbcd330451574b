"""Hazard check of the slot-ring schedule of the GEMM main loop (nmtgminor_amd/csrc/gemm_ring.hip.h).

A small event model of one wavefront replays the kernel's issue / wait / barrier / read sequence
with the kernel's own bookkeeping formulas (ring positions, number of transfers allowed to stay in
flight at each wait) and checks the three properties the loop relies on, for every ring size,
stage size and step count the templates admit:
  1. a slot is read only after its transfers were covered by a vmcnt wait that precedes the last
     barrier (transfers of a wavefront complete in issue order, `s_waitcnt vmcnt(n)` leaves at most
     the newest n outstanding; every wavefront runs the same sequence, so "covered before the
     barrier" for one holds for all);
  2. a ring position is overwritten only when the slot it held belongs to a stage every wavefront
     has finished reading (a barrier lies between the last read and the issue);
  3. the position arithmetic finds slot s * SPS + j of stage s where the kernel looks for it.
"""
import itertools

import pytest


def simulate(ring, sa, sb, ips, nk):
    sps = sa + sb
    assert ring >= 2 * sps
    total = nk * sps
    issued = []            # transfer ids in issue order: (slot number, instruction)
    content = [None] * ring  # slot number held (or being filled) at each ring position
    covered = set()        # slots whose transfers a wait has covered
    visible = set()        # ... and a barrier has followed

    def issue(q, pos, reading_stage):
        old = content[pos]
        if old is not None:
            # property 2: the slot being overwritten was consumed in an iteration that a barrier has closed
            assert old // sps < reading_stage, (ring, sps, nk, q, pos, old, reading_stage)
        content[pos] = q
        for i in range(ips):
            issued.append((q, i))

    def wait(n, max_n):
        k = min(n, max_n)
        assert k >= 0 and k % ips == 0
        done = issued if k == 0 else issued[:-k]
        for q, _ in done:
            covered.add(q)

    def barrier():
        visible.update(covered)

    def read_stage(st, pos):
        for j in range(sps):           # every operand slot of the stage is read by some wavefront
            p = pos + j
            if p >= ring:
                p -= ring
            q = st * sps + j
            assert content[p] == q, (ring, sps, nk, st, j, p, content[p])          # property 3
            assert q in visible, (ring, sps, nk, st, j)                             # property 1

    # prologue
    for t in range(ring):
        if t // sps < nk:
            issue(t, t, reading_stage=0)
    if nk > 0:
        wait((min(ring, total) - sps) * ips, (ring - sps) * ips)
    barrier()
    pos_r = pos_w = 0
    for s in range(nk):
        read_stage(s, pos_r)           # the first k-group's reads were issued behind the barrier of the step before
        pos_r += sps
        if pos_r >= ring:
            pos_r -= ring
        if s + 1 < nk:
            # in front of the last k-group's MFMAs: wait for stage s + 1, barrier, first reads of stage s + 1, and the
            # slots of stage s (all of its reads issued and landed before the barrier) are refilled
            n_issued = min(ring + s * sps, total)
            assert n_issued * ips == len(issued)
            wait((n_issued - (s + 2) * sps) * ips, (ring - 2 * sps) * ips)
            barrier()
            read_stage(s + 1, pos_r)
            for t in range(sps):
                d = (ring + t) // sps
                q = ring + s * sps + t
                assert q // sps == s + d and q % sps == (ring + t) % sps     # the kernel's compile-time (j, d)
                if s + d < nk:
                    issue(q, pos_w, reading_stage=s + 1)
                pos_w = 0 if pos_w + 1 == ring else pos_w + 1
    return len(issued)


def simulate_stepbuf(ring, sa, sb, ips, nk):
    """The loop form that keeps a whole stage's fragments in registers: phase p reads stage p (phase 0 ahead of the loop);
    a phase p >= 1 first multiplies, then waits for stage p, passes the barrier, refills the slots of stage p - 1 and
    reads stage p. Same three properties as simulate()."""
    sps = sa + sb
    assert ring >= 2 * sps
    total = nk * sps
    issued, content, covered, visible = [], [None] * ring, set(), set()
    done_reading = -1      # newest stage whose reads a barrier has closed

    def issue(q, pos):
        old = content[pos]
        if old is not None:
            assert old // sps <= done_reading, (ring, sps, nk, q, pos, old, done_reading)   # property 2
        content[pos] = q
        issued.extend((q, i) for i in range(ips))

    def wait(n, max_n):
        k = min(n, max_n)
        assert k >= 0 and k % ips == 0
        for q, _ in (issued if k == 0 else issued[:-k]):
            covered.add(q)

    def read_stage(st, pos):
        for j in range(sps):
            p = pos + j - (ring if pos + j >= ring else 0)
            q = st * sps + j
            assert content[p] == q, (ring, sps, nk, st, j, p, content[p])     # property 3
            assert q in visible, (ring, sps, nk, st, j)                        # property 1

    for t in range(ring):
        if t // sps < nk:
            issue(t, t)
    if nk > 0:
        wait((min(ring, total) - sps) * ips, (ring - sps) * ips)
    visible.update(covered)                                                   # barrier
    if nk == 0:
        return 0
    pos_r = pos_w = 0
    read_stage(0, pos_r)
    pos_r = (pos_r + sps) % ring
    for p in range(1, nk):
        n_issued = min(ring + (p - 1) * sps, total)
        assert n_issued * ips == len(issued)
        wait((n_issued - (p + 1) * sps) * ips, (ring - 2 * sps) * ips)
        visible.update(covered)                                               # barrier: also closes the reads of stage p - 1
        done_reading = p - 1
        for t in range(sps):
            d = (ring + t) // sps
            q = ring + (p - 1) * sps + t
            assert q // sps == p - 1 + d and q % sps == (ring + t) % sps
            if p - 1 + d < nk:
                issue(q, pos_w)
            pos_w = 0 if pos_w + 1 == ring else pos_w + 1
        read_stage(p, pos_r)
        pos_r = (pos_r + sps) % ring
    return len(issued)


CONFIGS = [(ring, sa, sb, ips) for ring, (sa, sb), ips in itertools.product((4, 5, 6, 8, 10), ((1, 1), (2, 1), (2, 2)), (2, 4))
           if ring >= 2 * (sa + sb)]


@pytest.mark.parametrize("ring,sa,sb,ips", CONFIGS)
def test_ring_schedule_has_no_hazard(ring, sa, sb, ips):
    for nk in range(0, 70):
        n = simulate(ring, sa, sb, ips, nk)
        assert n == nk * (sa + sb) * ips          # every slot of every stage is issued exactly once


@pytest.mark.parametrize("ring,sa,sb,ips", CONFIGS)
def test_ring_schedule_with_a_stage_of_fragments_in_registers_has_no_hazard(ring, sa, sb, ips):
    for nk in range(0, 70):
        n = simulate_stepbuf(ring, sa, sb, ips, nk)
        assert n == nk * (sa + sb) * ips


def test_shipped_configurations_are_covered():
    # 256x256 tile: 2 + 2 slots per stage, 10-slot ring, 8 wavefronts -> 2 transfers per wavefront and slot;
    # 128x128 tile: 1 + 1 slots, 5-slot ring, 4 wavefronts -> 4 transfers
    assert (10, 2, 2, 2) in CONFIGS and (5, 1, 1, 4) in CONFIGS
    # vmcnt is a 6-bit counter: the deepest wait the kernel can ask for must fit
    for ring, sa, sb, ips in ((10, 2, 2, 2), (5, 1, 1, 4)):
        assert (ring - (sa + sb)) * ips < 64
