"""A host-side model of the attention kernel's tile-load schedule (no GPU).

``attn_fwd_kernel`` (ditango_amd/csrc/attn_fwd.hip) brings K/V tiles into the LDS with loads the compiler
does not see; only hand-placed ``s_waitcnt vmcnt(N)`` and workgroup barriers order them against the LDS reads
of the two wavefront groups, which run one phase apart.  A wrong count does not fail a test reliably: the window
it opens is hit once in tens of thousands of work items.  So the schedule itself is checked here: the model
replays, for both groups, the sequence of load_tile calls (with their buffers), waits, barriers and LDS reads
that the kernel issues for a work item of ``n_tiles`` key tiles, with every constant taken from the table the
kernel itself is compiled from (ditango_amd/csrc/attn_schedule.h), and asserts

  (i)  every read of a buffer that expects tile X comes after a barrier that comes after, in EVERY wavefront
       group, a wait that covers that group's share of the loads of tile X;
  (ii) every load into a buffer is issued after a barrier that comes after the last read of the buffer's
       previous tile by any group, and after the same wavefront's earlier load into that buffer has landed;
  (iii) both groups pass the same number of barriers, and the epilogue (which reuses the tile buffers) starts
       behind a barrier behind every group's wait for all of its loads.

The order of the operations mirrors the kernel's control flow (prologue, the loop's vector and matrix phases,
epilogue); the COUNTS come from the table.  The model must reject the schedule without the trailing group's
explicit wait for K of tile 1 (the race that a 48-chunk parity case once showed) and accept the current one.
"""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TABLE = os.path.join(ROOT, "ditango_amd", "csrc", "attn_schedule.h")
KERNEL = os.path.join(ROOT, "ditango_amd", "csrc", "attn_fwd.hip")


def read_table(path=TABLE):
    """``{NAME: int}`` for every ``#define DT_SCHED_NAME <int>`` line of the shared header."""
    table = {}
    for line in open(path):
        m = re.match(r"\s*#define\s+DT_SCHED_([A-Z0-9_]+)\s+(-?\d+)\b", line)
        if m:
            table[m.group(1)] = int(m.group(2))
    return table


class Schedule:
    """The constants of one head dimension, in shares (one wavefront's loads of one operand of one tile)."""

    def __init__(self, table, D):
        s = "D64" if D == 64 else "D128"
        self.D = D
        self.num_buf = table["NUM_BUF"]
        self.loads_per_share = table[f"LOADS_{s}"]
        self.load_after_matrix = bool(table[f"LOAD_AFTER_MATRIX_{s}"])
        self.prologue_calls = (table["PROLOGUE_CALLS_LEADING"], table["PROLOGUE_CALLS_TRAILING"])
        self.call_ahead = table["CALL_AHEAD"]
        self.prologue_inflight = (table["PROLOGUE_INFLIGHT_LEADING"], table["PROLOGUE_INFLIGHT_TRAILING"])
        self.trailing_k1_inflight = table["TRAILING_K1_INFLIGHT"]      # None: the schedule without that wait
        self.vector_inflight = table[f"VECTOR_BARRIER_INFLIGHT_{s}"]


def wave_program(s: Schedule, group: int, n_tiles: int):
    """The operations one wavefront of ``group`` issues for a work item of ``n_tiles`` tiles, in program order:
    ("load", operand, tile, buffer) | ("wait", shares that may stay in flight) | ("barrier",) |
    ("read", operand, buffer, tile the reader expects) | ("epilogue",)."""
    ops = []

    def load_tile(y):
        # V of the tile before the load cursor first, then K of the tile under it (attn_fwd.hip: load_tile)
        ops.append(("load", "V", y - 1, (y - 1) % s.num_buf))
        ops.append(("load", "K", y, y % s.num_buf))

    # ---- prologue
    for y in range(s.prologue_calls[group]):
        load_tile(y)
    ops.append(("wait", s.prologue_inflight[group]))
    ops.append(("barrier",))
    if group == 1:
        ops.append(("barrier",))                      # the trailing group lets one phase pass
    if n_tiles > 0:
        ops.append(("read", "K", 0, 0))               # first matrix phase: scores of tile 0
    if group == 1 and s.trailing_k1_inflight is not None:
        ops.append(("wait", s.trailing_k1_inflight))
    ops.append(("barrier",))
    # ---- one iteration per tile: vector phase, then matrix phase
    for t in range(n_tiles):
        u = t % s.num_buf
        if not s.load_after_matrix:
            load_tile(t + s.call_ahead + group)
        ops.append(("read", "V", u, t))               # operand ring prefilled at the end of the vector phase
        ops.append(("wait", s.vector_inflight))
        ops.append(("barrier",))
        ops.append(("read", "V", u, t))               # P V of tile t
        ops.append(("read", "K", (u + 1) % s.num_buf, t + 1))   # scores of tile t + 1
        if s.load_after_matrix:
            load_tile(t + s.call_ahead + group)
        ops.append(("barrier",))
    # ---- epilogue: reuses the tile buffers
    ops.append(("wait", 0))
    if group == 0:
        ops.append(("barrier",))                      # the leading group waits out the phase it is ahead
    ops.append(("barrier",))
    ops.append(("epilogue",))
    return ops


def replay(s: Schedule, n_tiles: int):
    """Replays both groups.  Returns (violations, per-group facts).  An interval is the stretch between two
    barriers: operations of different groups in the same interval are concurrent."""
    facts = []
    for group in (0, 1):
        ops = wave_program(s, group, n_tiles)
        interval, issued = 0, []        # issued: [operand, tile, buffer, issue interval, landed-by interval or None]
        loads, reads, waw, epilogue_at, all_landed_at = [], [], [], None, None
        for op in ops:
            if op[0] == "barrier":
                interval += 1
            elif op[0] == "load":
                _, operand, tile, buf = op
                # the same wavefront's earlier load into this buffer must have landed (two loads never share a slot in flight)
                for rec in issued:
                    if rec[0] == operand and rec[2] == buf and rec[4] is None:
                        waw.append((group, operand, buf, rec[1], tile))
                issued.append([operand, tile, buf, interval, None])
            elif op[0] == "wait":
                # the counter retires in order: all but the newest `op[1]` shares have landed; the other wavefronts
                # see them behind the next barrier, i.e. from the next interval on
                for rec in issued[:max(0, len(issued) - op[1])]:
                    if rec[4] is None:
                        rec[4] = interval + 1
                if op[1] == 0:
                    all_landed_at = interval + 1
            elif op[0] == "read":
                reads.append((op[1], op[2], op[3], interval))
            elif op[0] == "epilogue":
                epilogue_at = interval
        loads = [tuple(r) for r in issued]
        facts.append(dict(barriers=interval, loads=loads, reads=reads, waw=waw, epilogue_at=epilogue_at,
                          all_landed_at=all_landed_at))
    bad = []
    if facts[0]["barriers"] != facts[1]["barriers"]:
        bad.append(("barrier count differs", facts[0]["barriers"], facts[1]["barriers"]))
    for g, f in enumerate(facts):
        for w in f["waw"]:
            bad.append(("load into a buffer whose previous load has not landed",) + w)
        # (i) reads of tiles that exist: every group's share must be visible
        for operand, buf, tile, at in f["reads"]:
            if tile >= n_tiles:
                continue                # scores computed past the last tile are never used
            for g2, f2 in enumerate(facts):
                mine = [l for l in f2["loads"] if l[0] == operand and l[1] == tile]
                if len(mine) != 1 or mine[0][2] != buf:
                    bad.append(("tile not loaded exactly once into the buffer it is read from", operand, tile, buf, g2))
                    continue
                visible = mine[0][4]
                if visible is None or visible > at:
                    bad.append((f"group {g} reads {operand} of tile {tile} in interval {at}, group {g2}'s share is visible from",
                                visible))
        # (ii) loads: the buffer's previous tile must have been read for the last time before the barrier in front of the issue
        for operand, tile, buf, at, _ in f["loads"]:
            for g2, f2 in enumerate(facts):
                for r_operand, r_buf, r_tile, r_at in f2["reads"]:
                    if r_operand == operand and r_buf == buf and r_tile < tile and r_tile < n_tiles and r_at >= at:
                        bad.append((f"group {g} loads {operand} of tile {tile} into buffer {buf} in interval {at} while group {g2} "
                                    f"still reads tile {r_tile} there in interval {r_at}",))
        # (iii) the epilogue overwrites every buffer
        for g2, f2 in enumerate(facts):
            if f2["all_landed_at"] is None or f2["all_landed_at"] > f["epilogue_at"]:
                bad.append((f"group {g}'s epilogue starts in interval {f['epilogue_at']}, group {g2}'s loads have all landed from",
                            f2["all_landed_at"]))
            for _, _, r_tile, r_at in f2["reads"]:
                if r_at >= f["epilogue_at"]:
                    bad.append((f"group {g}'s epilogue overlaps a tile read of group {g2} in interval {r_at}",))
    return bad, facts


TILE_COUNTS = list(range(0, 13)) + [35, 59, 233]      # short items (parts of split items are 6 tiles and up), the real shapes


@pytest.mark.parametrize("D", [128, 64])
def test_current_schedule_is_race_free(D):
    s = Schedule(read_table(), D)
    for n in TILE_COUNTS:
        bad, facts = replay(s, n)
        assert not bad, (D, n, bad[:3])
        # every tile that is read was loaded by both groups, K three and V two tiles ahead of its first use
        assert all(len(f["loads"]) == 2 * (s.prologue_calls[g] + n) for g, f in enumerate(facts))


@pytest.mark.parametrize("D", [128, 64])
def test_schedule_without_the_trailing_groups_wait_for_k1_is_rejected(D):
    """The leading group computes the scores of tile 1 while the trailing group has not ended a vector phase yet:
    without the trailing group's explicit wait, its share of K of tile 1 is not known to have landed."""
    s = Schedule(read_table(), D)
    s.trailing_k1_inflight = None
    for n in range(2, 13):
        bad, _ = replay(s, n)
        assert bad and any("reads K of tile 1" in str(b[0]) for b in bad), (D, n, bad[:3])
    bad, _ = replay(s, 1)          # a single tile never reads K of tile 1 for real
    assert not bad


@pytest.mark.parametrize("D", [128, 64])
def test_weaker_or_mistimed_waits_are_rejected(D):
    """The counts are tight: one more share in flight at any wait, one buffer fewer, or a call one tile further
    ahead opens a window the model sees."""
    base = read_table()
    suffix = "D64" if D == 64 else "D128"
    for key, delta in ((f"VECTOR_BARRIER_INFLIGHT_{suffix}", 1), ("PROLOGUE_INFLIGHT_LEADING", 1), ("PROLOGUE_INFLIGHT_TRAILING", 1),
                       ("TRAILING_K1_INFLIGHT", 1), ("NUM_BUF", -1), ("CALL_AHEAD", 1)):
        table = dict(base)
        table[key] += delta
        s = Schedule(table, D)
        assert any(replay(s, n)[0] for n in range(1, 13)), (D, key)


def test_kernel_takes_every_count_from_the_table():
    """No literal wait count, buffer count or call distance is left in the kernel source: it names the table's
    constants, so the model and the kernel cannot drift apart."""
    src = open(KERNEL).read()
    code = re.sub(r"//[^\n]*", "", src)
    assert '#include "attn_schedule.h"' in src
    for name in ("NUM_BUF", "LOADS_D128", "LOADS_D64", "LOAD_AFTER_MATRIX_D128", "LOAD_AFTER_MATRIX_D64", "PROLOGUE_CALLS_LEADING",
                 "PROLOGUE_CALLS_TRAILING", "CALL_AHEAD", "PROLOGUE_INFLIGHT_LEADING", "PROLOGUE_INFLIGHT_TRAILING",
                 "TRAILING_K1_INFLIGHT", "VECTOR_BARRIER_INFLIGHT_D128", "VECTOR_BARRIER_INFLIGHT_D64"):
        assert f"DT_SCHED_{name}" in code, name
        assert name in read_table(), name
    # waits are only ever written through the templated helpers, whose argument is a table expression
    literal_waits = re.findall(r'asm volatile\("s_waitcnt vmcnt\((\d+)\)', code)
    assert literal_waits == [], literal_waits
    for call in re.findall(r"wait_tile_loads<([^>]*)>", code):
        assert call.strip() in ("0", "N") or "DT_SCHED_" in call, call
    for call in re.findall(r"phase_barrier_after_vector<([^>]*)>", code):
        assert "kVectorInFlight" in call or "kInFlight" in call, call
    for call in re.findall(r"load_tile\(([^)]*)\)", code):
        assert call.strip() in ("y", "int kbuf") or "DT_SCHED_CALL_AHEAD" in call, call
