"""Model check of the decoupled look-back protocol of csrc/kernels/segscan.hip:
descriptor words {value, epoch, segment flag, status}; tiles numbered by a
ticket; a window of W descriptors per look-back step; tiles that contain a
segment start publish their prefix at once; 8-byte values travel as two words
which a reader accepts only when both carry the same meta word.

Every interleaving of the tiles' descriptor reads and writes is explored for a
few tiles (depth-first over global states), with at most R tiles resident at a
time and descriptor memory that starts out holding words of older launches.
Checked: no reachable state is stuck, and every tile ends with exactly the
exclusive prefix the sequential segmented scan gives it.  The operator is the
composition of affine maps modulo 7, which does not commute, so a fold in the
wrong order shows; in the two-word runs the two coefficients of a map travel
in different words, so a torn read would show as well.

This restates the protocol of the kernel; the reference's own is
src/Futhark/CodeGen/ImpGen/GPU/SegScan/SinglePass.hs:625-777 (status flags
X/A/P in an array of their own, fences between value and flag)."""
import itertools

import pytest

X, A, P = 0, 1, 2
IDENT = (1, 0)
EPOCH = 5


def op(f, g):
    """g after f for x -> a*x + b modulo 7 (associative, not commutative)."""
    return (f[0] * g[0] % 7, (g[0] * f[1] + g[1]) % 7)


def seg_apply(a, b):
    """The flag-tuple operator (Pass/Flatten/Builtins.hs:374-393) on (flag, value)."""
    return (a[0] | b[0], b[1] if b[0] else op(a[1], b[1]))


def expected_prefixes(aggs):
    out, acc = [], (0, IDENT)
    for agg in aggs:
        out.append(acc)
        acc = seg_apply(acc, agg)
    return out


def words_of(status, flag, value, words):
    """The descriptor words a publication writes, in the order it writes them."""
    meta = (EPOCH, flag, status)
    if words == 1:
        return [(meta, value)]
    return [(meta, value[0]), (meta, value[1])]


def tile_step(t, agg, state, mem, W, words, accept_torn=False):
    """One atomic step (at most one access to a descriptor word) of tile t's
    look-back program.  Returns (new_state, [(address, word)...]) or None when
    the step has to be retried later (nothing published yet)."""
    phase, sub, data = state
    flag, val = agg
    if phase == "publish":
        ws = words_of(P if (t == 0 or flag) else A, flag, val, words)
        after = ("done", 0, (0, IDENT)) if t == 0 else ("look", 0, (t - 1, (0, IDENT), (), None))
        nxt = ("publish", sub + 1, None) if sub + 1 < len(ws) else after
        return nxt, [((t, sub), ws[sub])]
    if phase == "look":
        j, acc, got, half = data  # newest tile of the window, fold so far, entries read, pending word 0
        tile = j - (W - 1) + len(got)
        if tile < 0:
            got, half = got + ((P, 0, IDENT),), None
        elif words == 1 or half is None:
            meta, v = mem[(tile, 0)]
            if meta[0] != EPOCH or meta[2] == X:
                return None  # the lane polls again
            if words == 1:
                got = got + ((meta[2], meta[1], v),)
            else:
                half = (meta, v)
        else:
            meta, v = mem[(tile, 1)]
            if meta != half[0] and not accept_torn:
                half = None  # halves of different publications: read the descriptor again
            elif meta[0] != EPOCH or meta[2] == X:
                return None
            else:
                got, half = got + ((meta[2], meta[1], (half[1], v)),), None
        if len(got) < W:
            new = ("look", 0, (j, acc, got, half))
            return (new, []) if new != state else None
        # the whole window is in: fold it as the kernel does, newest terminator restarts the fold
        term = [s == P or f == 1 for s, f, _ in got]
        first = max((l for l in range(W) if term[l]), default=None)
        win = (0, IDENT)
        for l in range(W):
            if first is None or l >= first:
                win = seg_apply(win, (got[l][1], got[l][2]))
        acc = seg_apply(win, acc)
        if first is None:
            return ("look", 0, (j - W, acc, (), None)), []
        if flag:  # this tile published its prefix at the start
            return ("done", 0, acc), []
        return ("prefix", 0, acc), []
    if phase == "prefix":
        inc = seg_apply(data, agg)
        ws = words_of(P, inc[0], inc[1], words)
        nxt = ("prefix", sub + 1, data) if sub + 1 < len(ws) else ("done", 0, data)
        return nxt, [((t, sub), ws[sub])]
    raise AssertionError(phase)


def explore(aggs, W, R, words, stale, accept_torn=False):
    """All interleavings, depth first; returns the number of states visited."""
    n = len(aggs)
    want = expected_prefixes(aggs)
    mem0 = {(i, w): stale[(i * words + w) % len(stale)] for i in range(n) for w in range(words)}
    start = (tuple(sorted(mem0.items())), (None,) * n, 0)  # memory, tile states, tickets drawn
    seen, stack = {start}, [start]
    while stack:
        mem_t, states, started = stack.pop()
        if all(s is not None and s[0] == "done" for s in states):
            for i, s in enumerate(states):
                assert s[2] == want[i], ("wrong prefix", aggs, i, s[2], want[i])
            continue
        mem = dict(mem_t)
        moves = []
        resident = sum(1 for s in states if s is not None and s[0] != "done")
        if started < n and resident < R:  # the next tile starts and draws the next ticket
            ns = list(states)
            ns[started] = ("publish", 0, None)
            moves.append((mem_t, tuple(ns), started + 1))
        for i, s in enumerate(states):
            if s is None or s[0] == "done":
                continue
            r = tile_step(i, aggs[i], s, mem, W, words, accept_torn)
            if r is None:
                continue
            ns, writes = r
            m2 = dict(mem)
            m2.update(writes)
            nstates = list(states)
            nstates[i] = ns
            moves.append((tuple(sorted(m2.items())), tuple(nstates), started))
        assert moves, ("stuck", aggs, states)
        for m in moves:
            if m not in seen:
                seen.add(m)
                stack.append(m)
    return len(seen)


VALUES = [(2, 3), (3, 1), (5, 6), (4, 4), (6, 2)]


def stale_words(words):
    """Descriptor memory left by older launches: every status, older epochs."""
    if words == 1:
        return [((4, 0, P), (3, 3)), ((3, 1, A), (2, 5)), ((0, 0, X), (0, 0))]
    return [((4, 0, P), 3), ((3, 1, A), 2), ((0, 0, X), 0), ((4, 1, P), 6)]


@pytest.mark.parametrize("words,n", [(1, 4), (2, 3)])
def test_every_interleaving_gives_the_sequential_prefixes(words, n):
    visited = 0
    for flags in itertools.product([0, 1], repeat=n):
        aggs = [(flags[i], VALUES[i]) for i in range(n)]
        for R in (1, 2, n):
            visited += explore(aggs, 2, R, words, stale_words(words))
    assert visited > 1000


def test_window_sizes_and_five_tiles():
    aggs = [(0, VALUES[i]) for i in range(3)]
    explore(aggs, 4, 1, 1, stale_words(1))          # window wider than the number of tiles
    explore(aggs, 1, 3, 1, stale_words(1))          # one descriptor per step
    explore([(f, VALUES[i]) for i, f in enumerate([0, 0, 1, 0, 0])], 2, 2, 1, stale_words(1))
    explore([(0, VALUES[i]) for i in range(5)], 3, 5, 1, stale_words(1))


def test_the_model_notices_a_broken_protocol():
    """The check has teeth: the operator does not commute, and a reader that
    accepts the two halves of a value from different publications is caught."""
    assert op((2, 3), (3, 1)) != op((3, 1), (2, 3))
    with pytest.raises(AssertionError, match="wrong prefix"):
        for flags in itertools.product([0, 1], repeat=3):
            explore([(flags[i], VALUES[i]) for i in range(3)], 2, 3, 2, stale_words(2),
                    accept_torn=True)


# ---------------------------------------------------------------------------
# Which ticket counter a persistent block draws from.
#
# The scan's blocks stay resident and draw tiles from several counters (counter
# c hands out the tiles congruent to c).  A block keeps one counter for its
# whole life and leaves when that counter has run out.  The model below
# explores every order in which the hardware may start blocks and in which the
# resident blocks take their steps, with at most R blocks resident, and asks
# whether a state is reachable from which nothing can move before all tiles are
# done.  Two rules for choosing the counter:
#   "arrival": the k-th block to START uses counter k mod C (the kernel's default);
#   "index":   block b uses counter b mod C, whatever the order of starts;
#   "static":  as "index", and the first two tiles of block b are b and b + G
#              without a ticket, the counters handing out tiles 2 G and up (what
#              the kernel does for callers that say the launch has the device to
#              itself).
def _ticket_model_deadlocks(rule, G, C, R, tiles):
    """True when some schedule gets stuck.  A block: take its next tile (by ticket from its
    counter, or by its index for the first two tiles under "static"); publish the tile's
    aggregate; look back (needs the aggregates of all earlier tiles); take the next.  It
    leaves on a tile beyond the last one."""
    base = 2 * G if rule == "static" else 0   # first tile the counters hand out

    # state: (counters, started mask, left mask, blocks, done mask) with blocks = tuple over
    # block ids of None (not started / left) or (counter, tiles taken, tile or None, published?)
    def moves(state):
        counters, started, left, blocks, done = state
        out = []
        resident = sum(b is not None for b in blocks)
        if resident < R:
            for b in range(G):
                if not (started >> b) & 1:
                    k = bin(started).count("1")
                    c = (k if rule == "arrival" else b) % C
                    nb = list(blocks)
                    nb[b] = (c, 0, None, False)
                    out.append((counters, started | (1 << b), left, tuple(nb), done))
                    if rule == "arrival":
                        break  # blocks are interchangeable until they have a counter
        for b, blk in enumerate(blocks):
            if blk is None:
                continue
            c, taken, tile, published = blk
            nb = list(blocks)
            if tile is None:  # take the next tile
                nc = list(counters)
                if rule == "static" and taken < 2:
                    t = b + taken * G
                    if t >= tiles:       # nothing here; the block goes on to its counter
                        nb[b] = (c, taken + 1, None, False)
                        out.append((counters, started, left, tuple(nb), done))
                        continue
                else:
                    t = base + counters[c] * C + c
                    nc[c] += 1
                if t >= tiles:
                    nb[b] = None
                    out.append((tuple(nc), started, left | (1 << b), tuple(nb), done))
                else:
                    nb[b] = (c, taken + 1, t, False)
                    out.append((tuple(nc), started, left, tuple(nb), done))
            elif not published:
                nb[b] = (c, taken, tile, True)
                out.append((counters, started, left, tuple(nb), done | (1 << tile)))
            elif done & ((1 << tile) - 1) == (1 << tile) - 1:  # every earlier aggregate is there
                nb[b] = (c, taken, None, False)
                out.append((counters, started, left, tuple(nb), done))
        return out

    start = ((0,) * C, 0, 0, (None,) * G, 0)
    seen, stack = {start}, [start]
    while stack:
        st = stack.pop()
        nxt = moves(st)
        finished = st[2] == (1 << G) - 1
        if not nxt and not finished:
            return True
        if finished:
            assert st[4] == (1 << tiles) - 1, "every tile was processed"
        for s in nxt:
            if s not in seen:
                seen.add(s)
                stack.append(s)
    return False


def test_counters_chosen_by_arrival_never_get_stuck():
    """With the counter chosen by arrival number, C resident blocks (or the whole grid) are
    enough for every schedule to finish; with the counter chosen by block index a grid that
    is not wholly resident can get stuck (the blocks that happen to run leave a counter
    without a drawer), and fewer than C resident blocks get stuck under either rule."""
    for G, C, tiles in ((4, 2, 7), (5, 2, 6), (6, 3, 8), (3, 3, 5)):
        for R in range(min(C, G), G + 1):
            assert not _ticket_model_deadlocks("arrival", G, C, R, tiles), (G, C, R)
        assert not _ticket_model_deadlocks("index", G, C, G, tiles)
        # the whole grid resident: the first two tiles may follow from the block index
        assert not _ticket_model_deadlocks("static", G, C, G, tiles)
        assert not _ticket_model_deadlocks("static", G, C, G, 2 * G + 3)
    assert _ticket_model_deadlocks("static", 4, 2, 3, 7)    # ... and only then
    assert _ticket_model_deadlocks("index", 4, 2, 2, 7)     # blocks 0 and 2 run: counter 1 starves
    assert _ticket_model_deadlocks("index", 6, 3, 4, 8)
    assert _ticket_model_deadlocks("arrival", 4, 2, 1, 7)   # the stated requirement is needed
