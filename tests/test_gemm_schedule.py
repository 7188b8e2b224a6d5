"""Work decomposition of the grouped GEMM, checked without a GPU through the library's introspection calls.

What must hold for ANY problem list, grid and tail-balancing choice (the kernel relies on each of these):
  * every (tile, K step) unit is processed exactly once; tiles without K work are visited exactly once;
  * an item is either a whole tile (slot -1) or a proper part of one with a workspace slot that no other
    item of the launch uses and that lies inside the kSlotsPerWg * grid slots of the workspace;
  * every tile that was cut is completed by exactly one fix-up workgroup, which adds exactly the slots
    written for that tile, in K order;
  * workgroup wg works only on tiles of XCD range wg % 8, and the eight ranges tile the list in order;
  * the tiles of a problem map one-to-one onto the 256 x 256 blocks of its output, and 32 consecutive tiles of
    a large problem form a compact block (at most 12 distinct row / column blocks), not a strip.
The expectations are stated from these properties, not recomputed with the scheduler's formulas.
"""
import numpy as np
import pytest

from fp8_gmm_amd import _lib

TILE = 256


def make_table(shapes):
    """shapes: list of (m, n, k). Pointers are fake but non-null and aligned; nothing is dereferenced."""
    t = np.zeros(len(shapes), dtype=_lib.GEMM_PROBLEM)
    for i, (m, n, k) in enumerate(shapes):
        t[i]["a"], t[i]["b"], t[i]["c"] = 0x10000, 0x20000, 0x30000
        t[i]["m"], t[i]["n"], t[i]["k"] = m, n, k
        t[i]["lda"] = t[i]["ldb"] = max(k, 16)
        t[i]["ldc"] = max(n, 1)
    total = _lib.plan_grouped_gemm(t)
    return t, total


def check_schedule(shapes, grid, stream_k):
    table, total = make_table(shapes)
    nk_of = [(k + 127) // 128 for (_, _, k) in shapes]
    tiles_of = [((m + TILE - 1) // TILE) * ((n + TILE - 1) // TILE) for (m, n, _) in shapes]
    assert total == sum(tiles_of)
    tile_prob = np.repeat(np.arange(len(shapes)), tiles_of)

    covered = [np.zeros(max(nk_of[p], 1), dtype=np.int32) for p in tile_prob]  # per tile, per K step
    slots_written = {}  # slot -> (tile, k_begin, nk)
    xcd_tiles = [set() for _ in range(8)]
    n_partial_items = 0
    origin_of = {}
    for wg in range(grid):
        items = _lib.gemm_schedule(table, total, grid, stream_k, wg)
        for tile, prob, m0, n0, k_begin, nk, slot in items.tolist():
            assert 0 <= tile < total and prob == tile_prob[tile]
            m, n, _ = shapes[prob]
            assert m0 % TILE == 0 and n0 % TILE == 0 and 0 <= m0 < m and 0 <= n0 < n
            origin_of.setdefault(tile, (prob, m0, n0))
            assert origin_of[tile] == (prob, m0, n0)   # every piece of a tile agrees on where the tile is
            xcd_tiles[wg % 8].add(tile)
            if nk_of[prob] == 0:
                assert (k_begin, nk, slot) == (0, 0, -1)
                covered[tile][0] += 1
                continue
            assert nk >= 1 and 0 <= k_begin and k_begin + nk <= nk_of[prob]
            covered[tile][k_begin:k_begin + nk] += 1
            if slot == -1:
                assert (k_begin, nk) == (0, nk_of[prob])
            else:
                assert stream_k and nk < nk_of[prob]
                assert 0 <= slot < 2 * grid and slot not in slots_written
                slots_written[slot] = (tile, k_begin, nk)
                n_partial_items += 1
    for tile in range(total):
        assert (covered[tile] == 1).all(), f"tile {tile} covered {covered[tile].tolist()}"
    # the tiles of a problem cover every 256 x 256 block of its output exactly once
    for p, (m, n, _) in enumerate(shapes):
        blocks = sorted((m0, n0) for (pp, m0, n0) in origin_of.values() if pp == p)
        want = sorted((i * TILE, j * TILE) for i in range((m + TILE - 1) // TILE) for j in range((n + TILE - 1) // TILE))
        assert blocks == want, f"problem {p}"
    # XCD ranges are disjoint, contiguous and ordered
    prev_end = 0
    for x in range(8):
        if xcd_tiles[x]:
            lo, hi = min(xcd_tiles[x]), max(xcd_tiles[x])
            assert lo == prev_end and xcd_tiles[x] == set(range(lo, hi + 1))
            prev_end = hi + 1
    assert prev_end == total

    # fix-up: each cut tile exactly once, with exactly its slots in K order
    cut_tiles = {}
    for slot, (tile, k_begin, nk) in slots_written.items():
        cut_tiles.setdefault(tile, []).append((k_begin, nk, slot))
    done = set()
    if stream_k and grid > 8:
        for wg in range(grid - 8):
            tile, slots = _lib.gemm_fixup(table, total, grid, wg)
            if tile < 0:
                assert slots == []
                continue
            assert tile in cut_tiles and tile not in done
            done.add(tile)
            pieces = sorted(cut_tiles[tile])
            assert slots == [s for (_, _, s) in pieces]
            # the pieces tile the K range of the tile without gaps
            pos = 0
            for k_begin, nk, _ in pieces:
                assert k_begin == pos
                pos += nk
            assert pos == nk_of[tile_prob[tile]]
    assert done == set(cut_tiles)
    check_launch_plan(shapes, table, total, grid, stream_k)
    return n_partial_items


def check_launch_plan(shapes, table, total, grid, stream_k):
    """The work list the kernels read (fp8gmm_plan_grouped_gemm_launch) is the schedule above written out:
    record r of workgroup w sits at items[r * grid + w], lists end with prob == -1, the slots of a shared
    tile are consecutive in K order, and every record carries the addresses and extents of its tile's operands."""
    plan, items, fixups = _lib.plan_grouped_gemm_launch(table.copy(), 0, grid, stream_k)
    assert plan.total_tiles == total
    if total == 0:
        return
    sk = stream_k and total <= 24 * grid and grid > 8
    g = plan.grid
    assert g == (grid if sk else min(grid, (total + 7) // 8 * 8)) and len(items) == plan.rounds * g
    items = items.reshape(plan.rounds, g)
    slot_name = {}      # uncompacted slot -> slot of the plan
    pieces_of = {}      # (prob, m0, n0) -> [(k_begin, plan slot)]
    longest = 0
    for wg in range(g):
        want = _lib.gemm_schedule(table, total, g, sk, wg).tolist()
        longest = max(longest, len(want))
        col = items[:, wg]
        assert (col["prob"][len(want):] == -1).all() and len(want) < plan.rounds
        for rec, (tile, prob, m0, n0, k_begin, nk, slot) in zip(col, want):
            assert (rec["prob"], rec["m0"], rec["n0"], rec["k_begin"], rec["nk"]) == (prob, m0, n0, k_begin, nk)
            m, n, k = shapes[prob]
            lda = ldb = max(k, 16)
            assert (rec["k"], rec["lda"], rec["ldb"]) == (k, lda, ldb)
            if k > 0:
                assert rec["a"] == 0x10000 + m0 * lda and rec["b"] == 0x20000 + n0 * ldb
                assert rec["a_bytes"] == (min(m - m0, TILE) - 1) * lda + k
                assert rec["b_bytes"] == (min(n - n0, TILE) - 1) * ldb + k
            if slot < 0:
                assert rec["slot"] == -1
            else:
                assert 0 <= rec["slot"] < plan.n_slots and slot not in slot_name
                slot_name[slot] = int(rec["slot"])
                pieces_of.setdefault((prob, m0, n0), []).append((k_begin, int(rec["slot"])))
        # height: whole tiles with at most 128 valid rows are flagged; a record without K steps repeats, one bit
        # up, the flag of the workgroup's next record that has some
        following = 0
        for rec, (tile, prob, m0, n0, k_begin, nk, slot) in reversed(list(zip(col, want))):
            half = int(slot < 0 and shapes[prob][0] - m0 <= TILE // 2)
            if nk == 0:
                assert rec["flags"] == half | following << 1
            else:
                assert rec["flags"] == half
                following = half
    assert plan.rounds == longest + 1
    assert sorted(slot_name.values()) == list(range(plan.n_slots))   # renumbered from 0 without gaps
    assert plan.n_fixups == len(fixups) == len(pieces_of)
    seen = set()
    for f in fixups:
        key = (int(f["prob"]), int(f["m0"]), int(f["n0"]))
        assert key in pieces_of and key not in seen
        seen.add(key)
        slots_in_k_order = [s for _, s in sorted(pieces_of[key])]
        assert slots_in_k_order == list(range(f["first_slot"], f["first_slot"] + f["n_pieces"]))


def test_launch_plan_of_contraction_major_operands():
    """Addresses and extents of the records when operands are stored contraction-major (gradient GEMMs)."""
    t = np.zeros(2, dtype=_lib.GEMM_PROBLEM)
    t["a"], t["b"], t["c"] = 0x10000, 0x20000, 0x30000
    t["m"], t["n"], t["k"] = [512, 272], [768, 768], [300, 77]
    t["lda"], t["ldb"], t["ldc"] = [512, 288], [768, 800], 768
    for layout in (_lib.GEMM_B_KMAJOR, _lib.GEMM_B_KMAJOR | _lib.GEMM_A_KMAJOR):
        tt = t.copy()
        if not layout & _lib.GEMM_A_KMAJOR:
            tt["k"] = tt["lda"] = [304, 80]   # a is [m, k] here, fetched in 16-byte pieces of k
        plan, items, _ = _lib.plan_grouped_gemm_launch(tt, layout, 16, False)
        recs = items[items["prob"] >= 0]
        assert len(recs) == plan.total_tiles == 2 * 3 + 2 * 3
        for r in recs:
            p = int(r["prob"])
            m, n, k, lda, ldb = (int(tt[f][p]) for f in ("m", "n", "k", "lda", "ldb"))
            assert r["b"] == 0x20000 + r["n0"] and r["b_bytes"] == (k - 1) * ldb + (n - r["n0"])
            if layout & _lib.GEMM_A_KMAJOR:
                assert r["a"] == 0x10000 + r["m0"] and r["a_bytes"] == (k - 1) * lda + (m - r["m0"])
            else:
                assert r["a"] == 0x10000 + r["m0"] * lda and r["a_bytes"] == (min(m - r["m0"], 256) - 1) * lda + k


MLP = [1439, 3146, 3993, 1820, 909, 3499, 669, 909]


@pytest.mark.parametrize("grid", [256, 64, 8])
@pytest.mark.parametrize("stream_k", [False, True])
def test_config2_shapes(grid, stream_k):
    fc1 = [(m, 14336, 4096) for m in MLP]
    fc2 = [(m, 4096, 14336) for m in MLP]
    wgrad = [(14336, 4096, (m + 127) // 128 * 128) for m in MLP]
    check_schedule(fc1, grid, stream_k)
    n_cut = check_schedule(fc2, grid, stream_k)
    check_schedule(wgrad, grid, stream_k)
    if stream_k and grid == 256:
        # 1088 tiles on 256 workgroups: 4.25 rounds, so the tail must be shared along K
        assert n_cut > 0


def test_tail_balancing_is_off_when_it_cannot_pay():
    # 28 full rounds: more than the limit, nothing may be cut
    assert check_schedule([(14336, 4096, 2048)] * 8, 256, True) == 0
    # an exact multiple of the grid: no remainder
    assert check_schedule([(2048, 4096, 4096)] * 8, 256, True) == 0


@pytest.mark.parametrize("shapes", [
    [(1, 1, 16)],
    [(256, 256, 128)],
    [(256, 256, 4096)],                      # one tile, cut eight ways at most
    [(300, 520, 1040)],
    [(0, 128, 64), (128, 0, 64), (64, 64, 0), (100, 100, 4096)],   # empty problems, a problem without K
    [(137, 64, 128), (401, 64, 128), (59, 64, 128), (403, 64, 128)],
    [(2048, 4096, 14336)],
    [(513, 777, 1616), (31, 2049, 48), (1025, 255, 8192)],
])
@pytest.mark.parametrize("grid", [256, 32, 8])
def test_small_and_odd_shapes(shapes, grid):
    check_schedule(shapes, grid, False)
    check_schedule(shapes, grid, True)


def test_random_problem_lists():
    rng = np.random.default_rng(1234)
    for _ in range(150):
        e = int(rng.integers(1, 12))
        shapes = []
        for _ in range(e):
            m = int(rng.choice([0, 1, 100, 256, 257, 700, 1500, 4000]))
            n = int(rng.choice([0, 16, 256, 1000, 4096]))
            k = int(rng.choice([0, 16, 128, 144, 1024, 4096, 14336]))
            shapes.append((m, n, k))
        grid = int(rng.choice([8, 16, 64, 256, 304]))
        check_schedule(shapes, grid, bool(rng.integers(0, 2)))


def test_argument_checks():
    table, total = make_table([(256, 256, 128)])
    buf = np.zeros((4, 7), dtype=np.int32)
    L = _lib.load()
    assert L.fp8gmm_gemm_schedule(table.ctypes.data, 1, total, 12, 1, 0, buf.ctypes.data, 4) < 0   # grid % 8 != 0
    assert L.fp8gmm_gemm_schedule(table.ctypes.data, 1, total, 16, 1, 16, buf.ctypes.data, 4) < 0  # wg out of range
    assert L.fp8gmm_gemm_schedule(None, 1, total, 16, 1, 0, buf.ctypes.data, 4) < 0


def test_consecutive_tiles_form_compact_blocks():
    """One round of an XCD is 32 consecutive tiles: they must touch few distinct operand slabs (8 row blocks +
    4 column blocks), also for weight-gradient shapes with many more row blocks than column blocks."""
    for shape in [(14336, 4096, 2048), (4096, 14336, 2048), (2048, 14336, 4096)]:
        table, total = make_table([shape])
        tiles = {}
        for wg in range(256):
            for tile, _, m0, n0, *_ in _lib.gemm_schedule(table, total, 256, False, wg).tolist():
                tiles[tile] = (m0, n0)
        for start in range(0, total - 31, 32):
            rows = {tiles[t][0] for t in range(start, start + 32)}
            cols = {tiles[t][1] for t in range(start, start + 32)}
            assert len(rows) + len(cols) <= 12, (shape, start, len(rows), len(cols))


@pytest.mark.parametrize("flag,tm,tn", [(_lib.GEMM_TILE_128, 128, 128), (_lib.GEMM_TILE_DUAL, 128, 256)])
def test_whole_tile_plans(flag, tm, tn):
    """FP8GMM_GEMM_TILE_128 / FP8GMM_GEMM_TILE_DUAL: the same launch cut into 128 x 128 / 128 x 256 tiles, whole tiles
    only.  Every such block of every output exactly once, records with the addresses and extents of a slab of that
    many rows / columns, XCD ranges contiguous and in order, no workspace, no fix-up launch; not available together
    with the GELU epilogue."""
    rng = np.random.default_rng(7)
    cases = [[(137, 512, 256), (401, 512, 256), (0, 512, 256), (59, 512, 256)],
             [(64, 1408, 2048)] * 64,
             [(1, 16, 16)],
             [(300, 520, 1040), (129, 128, 0), (128, 129, 4096)]]
    for _ in range(20):
        cases.append([(int(rng.choice([0, 1, 100, 128, 129, 300, 700])), int(rng.choice([16, 128, 144, 1000])),
                       int(rng.choice([0, 16, 128, 1040, 4096]))) for _ in range(int(rng.integers(1, 10)))])
    for shapes in cases:
        for layout in (0, _lib.GEMM_B_KMAJOR, _lib.GEMM_B_KMAJOR | _lib.GEMM_A_KMAJOR):
            t = np.zeros(len(shapes), dtype=_lib.GEMM_PROBLEM)
            for i, (m, n, k) in enumerate(shapes):
                if layout & _lib.GEMM_A_KMAJOR:
                    m = (m + 15) // 16 * 16
                if layout & _lib.GEMM_B_KMAJOR:
                    n = (n + 15) // 16 * 16
                t[i]["a"], t[i]["b"], t[i]["c"] = 0x10000, 0x20000, 0x30000
                t[i]["m"], t[i]["n"], t[i]["k"] = m, n, k
                t[i]["lda"] = max(m if layout & _lib.GEMM_A_KMAJOR else k, 16)
                t[i]["ldb"] = max(n if layout & _lib.GEMM_B_KMAJOR else k, 16)
                t[i]["ldc"] = max(n, 1)
            grid = 512
            plan, items, fixups = _lib.plan_grouped_gemm_launch(t.copy(), layout | flag, grid, True)
            want = {(p, i * tm, j * tn) for p in range(len(t))
                    for i in range((int(t["m"][p]) + tm - 1) // tm) for j in range((int(t["n"][p]) + tn - 1) // tn)}
            assert plan.tile == tn and plan.tile_m == (0 if tm == tn else tm)
            assert plan.total_tiles == len(want) and plan.n_slots == 0 and plan.n_fixups == 0
            assert len(fixups) == 0
            if not want:
                continue
            assert plan.grid == min(grid, (len(want) + 7) // 8 * 8) and len(items) == plan.rounds * plan.grid
            items = items.reshape(plan.rounds, plan.grid)
            seen, order = set(), {}
            for wg in range(plan.grid):
                col = items[:, wg]
                count = int((col["prob"] >= 0).sum())
                assert (col["prob"][:count] >= 0).all() and (col["prob"][count:] == -1).all() and count < plan.rounds
                for r in col[:count]:
                    p, m0, n0 = int(r["prob"]), int(r["m0"]), int(r["n0"])
                    m, n, k, lda, ldb = (int(t[f][p]) for f in ("m", "n", "k", "lda", "ldb"))
                    assert (p, m0, n0) in want and (p, m0, n0) not in seen
                    seen.add((p, m0, n0))
                    order.setdefault(wg % 8, []).append(p)
                    assert (r["k_begin"], r["nk"], r["slot"], r["k"]) == (0, (k + 127) // 128, -1, k)
                    if k > 0:
                        if layout & _lib.GEMM_A_KMAJOR:
                            assert r["a"] == 0x10000 + m0 and r["a_bytes"] == (k - 1) * lda + (m - m0)
                        else:
                            assert r["a"] == 0x10000 + m0 * lda and r["a_bytes"] == (min(m - m0, tm) - 1) * lda + k
                        if layout & _lib.GEMM_B_KMAJOR:
                            assert r["b"] == 0x20000 + n0 and r["b_bytes"] == (k - 1) * ldb + (n - n0)
                        else:
                            assert r["b"] == 0x20000 + n0 * ldb and r["b_bytes"] == (min(n - n0, tn) - 1) * ldb + k
            assert seen == want
            # the XCD ranges follow the problem order
            last = -1
            for x in range(8):
                if x in order:
                    assert min(order[x]) >= last
                    last = max(order[x])
    # no fused GELU epilogue with these tiles, and one tile flag at a time
    t, _ = make_table([(256, 256, 128)])
    import ctypes
    plan = _lib.GemmPlan()
    for bad in (flag | _lib.EPI_GELU, _lib.GEMM_TILE_128 | _lib.GEMM_TILE_DUAL):
        assert _lib.load().fp8gmm_plan_grouped_gemm_launch(t.ctypes.data, 1, bad, 16, 0, None, 0, None, 0,
                                                           ctypes.byref(plan)) < 0


def test_half_height_flag_marks_the_ragged_last_row_of_tiles():
    """FP8GMM_ITEM_HALF_HEIGHT: the one tile row of a 100-row problem and the last of a 300-row problem (44 rows),
    not the 129 valid rows of a 385-row problem; never a piece of a tile shared along K; never a 128 x 128 tile."""
    shapes = [(100, 512, 256), (300, 512, 256), (385, 256, 256), (128, 256, 256)]
    table, total = make_table(shapes)
    plan, items, _ = _lib.plan_grouped_gemm_launch(table.copy(), 0, 8, False)
    recs = items[items["prob"] >= 0]
    assert len(recs) == total == 2 + 4 + 2 + 1
    flagged = sorted((int(r["prob"]), int(r["m0"]), int(r["n0"])) for r in recs if r["flags"] & 1)
    assert flagged == [(0, 0, 0), (0, 0, 256), (1, 256, 0), (1, 256, 256), (3, 0, 0)]
    assert (items["flags"][items["prob"] < 0] == 0).all()
    # a single short tile, shared along K between the workgroups: pieces run at full height
    table, total = make_table([(100, 256, 8192)])
    plan, items, fixups = _lib.plan_grouped_gemm_launch(table.copy(), 0, 64, True)
    assert plan.n_slots > 1 and len(fixups) == 1 and (items["flags"] == 0).all()
    plan, items, _ = _lib.plan_grouped_gemm_launch(table.copy(), _lib.GEMM_TILE_128, 64, False)
    assert plan.tile == 128 and (items["flags"] == 0).all()


def test_slot_cap_falls_back_to_whole_tiles():
    """stream_k > 1 states how many workspace slots the caller has: a plan that would need more shares nothing."""
    fc2 = [(m, 4096, 14336) for m in MLP]
    table, total = make_table(fc2)
    free, items_free, fix_free = _lib.plan_grouped_gemm_launch(table.copy(), 0, 256, True)
    assert free.n_slots > 2 and free.n_fixups > 0
    enough, items_enough, fix_enough = _lib.plan_grouped_gemm_launch(table.copy(), 0, 256, free.n_slots)
    assert (enough.n_slots, enough.n_fixups, enough.rounds) == (free.n_slots, free.n_fixups, free.rounds)
    assert items_enough.tobytes() == items_free.tobytes() and fix_enough.tobytes() == fix_free.tobytes()
    whole, items_whole, _ = _lib.plan_grouped_gemm_launch(table.copy(), 0, 256, False)
    short, items_short, fix_short = _lib.plan_grouped_gemm_launch(table.copy(), 0, 256, free.n_slots - 1)
    assert (short.n_slots, short.n_fixups, len(fix_short)) == (0, 0, 0) and short.rounds == whole.rounds
    assert items_short.tobytes() == items_whole.tobytes()
