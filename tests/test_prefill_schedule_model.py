"""Happens-before model of the persistent prefill consumer's schedule (CPU only; nothing runs on a GPU).

`sparse_attn_prefill_kernel` (moespresso_amd/csrc/sparse_attn.hip) streams the 32-slot tiles of consecutive
(token, head block) units through a ring of four LDS buffers and prepares the next unit inside the current unit's
tile loop. Every wave of the workgroup runs the same program, so two actions of different waves are ordered only
if a workgroup barrier lies between them: an action's epoch is the number of barriers passed before it, and
"X before Y in every interleaving" means epoch(X) < epoch(Y). This file replays the order of actions of that
program (the list in `program` mirrors the kernel's source order, step by step) for random unit lengths and random
flagged tiles and checks

* every LDS resource that one wave writes and another reads (tile ring, row-pointer tables and validity words,
  stop positions, P^T, flags, the maximum and denominator exchanges) has its writes and reads in different epochs,
  in the right order, and is not rewritten while the previous contents may still be read;
* the vector-memory wait counts: a wave's `s_waitcnt vmcnt(issued - mark)` may leave at most as many operations in
  flight as were really issued behind the awaited request (operations complete in issue order), with the
  compiler-visible loads and stores that the count leaves out or includes modelled as the kernel has them.
"""

import itertools
import random

K_MINE = 5          # asynchronous copies of one wave per tile (4 in the waves that skip the last round)
MIN_TILES = 5       # PrefillGeometry::kMinTiles


def wait_level(n):
    """What `wait_vm_dyn(n)` really passes to vmcnt: the largest of its levels that does not exceed n."""
    if n in (4, 5):
        return n
    if n >= 20:
        return 20
    return 6 if n >= 6 else 0


def program(units, flagged, have_ids=True, stores_counted=None, copies_counted=None, early_min_t=3):
    """Events of one wave: (epoch, kind, payload...) in program order, plus the vector-memory log (tags in issue
    order) and the waits [(position in the log of the awaited operation, n passed to vmcnt, operations issued by
    then, what)]. `stores_counted` is what the wave adds to its count per unit for the output stores (the kernel:
    sixteen, as many as every wave issues), `copies_counted` what it adds per tile (the kernel: the copies it
    issues)."""
    ev, epoch = [], 0
    vm, waits = [], []
    if stores_counted is None:
        stores_counted = 16
    if copies_counted is None:
        copies_counted = K_MINE
    issued = 0
    marks = {}

    def bar():
        nonlocal epoch
        epoch += 1

    def act(kind, *p):
        ev.append((epoch, kind) + p)

    def issue(tag, n, counted):
        nonlocal issued
        for _ in range(n):
            vm.append(tag)
        if counted:
            issued += copies_counted if tag[0] == "tile" else n

    def tile_sources(flat):
        act("table_read", unit_of[flat])

    def issue_copies(flat):
        act("copy", flat)
        issue(("tile", flat), K_MINE, True)
        marks[("tile", flat % 4)] = (issued, len(vm) - 1)

    def copy_tile(flat):
        tile_sources(flat)
        issue_copies(flat)

    def await_tile(flat):
        mark, pos = marks[("tile", flat % 4)]
        waits.append((pos, wait_level(issued - mark), len(vm), ("tile", flat)))
        act("await", flat)

    def request_ids(u):
        act("ids_request", u)
        issue(("ids", u), 2, True)
        marks["ids"] = (issued, len(vm) - 1)

    def await_ids(u):
        mark, pos = marks["ids"]
        waits.append((pos, wait_level(issued - mark), len(vm), ("ids", u)))
        act("ids_read", u)

    total = sum(units)
    unit_of = [u for u, n in enumerate(units) for _ in range(n)]
    t_of = [t for n in units for t in range(n)]

    # ---- prologue (first unit)
    if have_ids:
        request_ids(0)
    issue(("q", 0), 16, False)            # ordinary loads: not counted
    act("stop_init", 0)
    bar()                                  # __syncthreads
    if have_ids:
        await_ids(0)
        act("stop_scan", 0)
    bar()                                  # __syncthreads
    act("stop_read", 0)
    act("table_build", 0)
    waits.append((len(vm) - 1, 0, len(vm), ("q", 0)))     # await_q: the compiler's own wait, nothing issued since
    issue(("sink", 0), 1, False)
    waits.append((len(vm) - 1, 0, len(vm), ("sink", 0)))
    bar()                                  # __syncthreads
    for j in range(min(3, total)):
        copy_tile(j)
    await_tile(0)
    bar()
    act("qk", 0)

    s = 0
    for u, n in enumerate(units):
        have_next = u + 1 < len(units)
        for t in range(n):
            last = t == n - 1
            if have_next:
                if t == 1 and have_ids:
                    await_ids(u + 1)
                    act("stop_scan", u + 1)
                if t == 0:
                    if have_ids:
                        request_ids(u + 1)
                    act("stop_init", u + 1)
                if t == 2:
                    issue(("warm", u + 1), 1, True)
            # row pointers of tile s+3: read here unless they are the next unit's and t < 3
            ahead = s + 3 < total and (t + 3 < n or have_next)
            early = ahead and (t + 3 < n or t >= early_min_t)
            if early:
                tile_sources(s + 3)
            act("vmask_read", u)
            act("p_write", s)
            if s in flagged:
                act("flag_write", s)
            if not last or have_next:
                await_tile(s + 1)
            bar()                          # C
            act("flag_read", s)
            if ahead:
                if not early:
                    tile_sources(s + 3)
                issue_copies(s + 3)
            if s in flagged:
                act("tmax_write", s)
                bar()
                act("tmax_read", s)
                act("p_write", s)
                bar()
            if have_next and t == 1:
                act("stop_read", u + 1)
                act("table_build", u + 1)
            if not last:
                act("p_read", s)
                act("pv", s)
                act("qk", s + 1)
            s += 1
        # ---- end of the unit: the next unit's query rows are requested, then the last tile is multiplied
        if have_next:
            issue(("q", u + 1), 16, False)
        act("p_read", s - 1)
        act("pv", s - 1)
        act("l_write", u)
        bar()
        act("l_read", u)
        issue(("store", u), 16, False)       # issued by the compiler, every lane active (lanes without a head
                                             # store into a sink)
        if have_next:
            # await_q: the compiler waits for the query loads; it may leave its own younger stores in flight
            qpos = max(i for i, tag in enumerate(vm) if tag == ("q", u + 1))
            waits.append((qpos, len(vm) - 1 - qpos, len(vm), ("q", u + 1)))
        issued += stores_counted             # the wave's own count of those stores
        if not have_next:
            break
        act("qk", s)
    return ev, epoch, vm, waits


def epochs(ev, kind, *p):
    return [e for (e, k, *q) in ev if k == kind and tuple(q) == p]


def check(units, flagged, **kw):
    ev, n_bar, vm, waits = program(units, flagged, **kw)
    total = sum(units)
    # ---- vector-memory waits: vmcnt(n) completes everything but the n youngest operations, so the awaited one
    #      is complete iff at least n operations were issued behind it
    for pos, n, issued_by_then, what in waits:
        younger = issued_by_then - 1 - pos
        assert 0 <= n <= younger, ("a wait leaves more in flight than was issued behind the request", what, n, younger)
    # ---- tile ring
    for j in range(total):
        readers = epochs(ev, "qk", j) + epochs(ev, "pv", j)
        assert readers, j
        aw = epochs(ev, "await", j)
        cp = epochs(ev, "copy", j)
        assert len(cp) == 1 and len(aw) == 1 and cp[0] <= aw[0], ("copy / await", j)
        assert aw[0] < min(readers), ("tile read before every wave has waited for its copies", j)
        if j >= 4:
            old = epochs(ev, "qk", j - 4) + epochs(ev, "pv", j - 4)
            assert cp[0] > max(old), ("copy into a ring buffer that is still being read", j)
    # ---- per-unit preparation
    for u in range(len(units)):
        builds, reads = epochs(ev, "table_build", u), epochs(ev, "table_read", u) + epochs(ev, "vmask_read", u)
        assert len(builds) == 1 and reads and builds[0] < min(reads), ("table read before it is built", u)
        inits, scans, sreads = epochs(ev, "stop_init", u), epochs(ev, "stop_scan", u), epochs(ev, "stop_read", u)
        assert len(inits) == 1 and len(sreads) == 1
        if scans:
            assert inits[0] < scans[0] < sreads[0], ("stop position", u)
        if u >= 2:   # the same table / stop slot held unit u-2
            old = epochs(ev, "table_read", u - 2) + epochs(ev, "vmask_read", u - 2)
            assert max(old) < builds[0], ("table slot rewritten while still read", u)
            assert epochs(ev, "stop_read", u - 2)[0] < inits[0], ("stop slot rewritten while still read", u)
        lw, lr = epochs(ev, "l_write", u), epochs(ev, "l_read", u)
        assert lw[0] < lr[0]
        if u >= 1:
            assert epochs(ev, "l_read", u - 1)[0] < lw[0], ("denominator exchange rewritten while still read", u)
    # ---- per-step exchanges
    for s in range(total):
        w, r = epochs(ev, "p_write", s), epochs(ev, "p_read", s)
        assert max(w) < r[0], ("P^T read before it is written", s)
        if s >= 2:
            assert epochs(ev, "p_read", s - 2)[0] < min(w), ("P^T rewritten while still read", s)
        fr = epochs(ev, "flag_read", s)[0]
        fw = epochs(ev, "flag_write", s)
        if fw:
            assert fw[0] < fr
        if s >= 2:
            assert epochs(ev, "flag_read", s - 2)[0] < (fw[0] if fw else fr), ("flag rewritten while still read", s)
        tw, tr = epochs(ev, "tmax_write", s), epochs(ev, "tmax_read", s)
        if tw:
            assert tw[0] < tr[0]
    flagged_steps = sorted(s for s in flagged if s < total)
    for a, b in zip(flagged_steps, flagged_steps[1:]):
        assert epochs(ev, "tmax_read", a)[0] < epochs(ev, "tmax_write", b)[0], ("maximum exchange rewritten early", b)
    return n_bar


def test_schedule_keeps_every_shared_resource_race_free_and_every_wait_sufficient():
    rng = random.Random(1)
    for _ in range(120):
        units = [rng.randint(MIN_TILES, 22) for _ in range(rng.randint(1, 6))]
        total = sum(units)
        firsts = set(itertools.accumulate([0] + units[:-1]))     # a unit's first tile always raises the flag
        flagged = firsts | {s for s in range(total) if rng.random() < 0.2}
        check(units, flagged, have_ids=rng.random() < 0.8)


def test_every_tile_flagged_and_shortest_units():
    check([MIN_TILES] * 4, set(range(4 * MIN_TILES)))
    check([MIN_TILES], {0})
    check([22, MIN_TILES, 22], {0, 22, 27})


def test_the_model_sees_a_wait_that_is_too_short():
    """Counting operations that were never issued ends a wait early; the model must report it. (Phantom stores
    would not: with the stores in flight the wait is for twenty, and the sixteen query loads that the count leaves
    out sit at the same place.)"""
    import pytest

    check([6, 6, 6], {0, 6, 12})
    check([6, 6, 6], {0, 6, 12}, stores_counted=40)
    with pytest.raises(AssertionError, match="more in flight"):
        check([6, 6, 6], {0, 6, 12}, copies_counted=K_MINE + 1)


def test_the_model_sees_row_pointers_read_too_early():
    """The next unit's row pointers are written behind the barrier of step 1; reading them at the top of step 2
    (which a unit of five tiles would do for its tile 5 = the next unit's tile 0) has no barrier in between."""
    import pytest

    check([5, 5, 5], {0, 5, 10})
    with pytest.raises(AssertionError, match="table read before it is built"):
        check([5, 5, 5], {0, 5, 10}, early_min_t=2)


def test_wait_levels_never_exceed_the_count():
    for n in range(0, 64):
        assert 0 <= wait_level(n) <= n
    assert [wait_level(n) for n in (4, 5, 6, 7, 10, 21, 23)] == [4, 5, 6, 6, 6, 20, 20]


def test_the_model_sees_a_ring_that_is_too_shallow():
    """A copy three tiles ahead into a ring of three buffers would overwrite the tile under V^T.P^T."""
    import pytest

    ev, _, _, _ = program([8], {0})
    copies = {p[0]: e for (e, k, *p) in ev if k == "copy"}
    pv = {p[0]: e for (e, k, *p) in ev if k == "pv"}
    # with four buffers tile j+4 replaces tile j: its copy is issued after the last read of tile j ...
    assert all(copies[j + 4] > pv[j] for j in range(4))
    # ... with three it would replace tile j+1, which is read in the same epoch as the copy is issued
    assert any(copies[j + 3] <= pv[j] for j in range(1, 5) if j + 3 in copies)
