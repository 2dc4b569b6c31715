"""Invariants of the static GEMM plan (tile order, beta schedule, block assignment, dependency edges), checked on
the host, and a pure-Python replay of the plan on integer data against numpy."""
import itertools

import numpy as np
import pytest

FETCH_A, FETCH_B, FETCH_C, GEMM, REDUCE, WRITEBACK = range(6)
BETA_ZERO, BETA_ONE, BETA_USER = 0, 1, 2
H2D, D2H, EXEC0 = 0, 1, 2
K_AXIS = object()   # marks a slice request along k, whose tiles need not be uniform


def kbounds(K, T, slabs=1):
    """First k of every k tile, and K: tiles of T, the first one cut by a thin start (order ids of 160000 and above) when
    K >= T and the slabs are whole and at least 16 deep: slabs = 2 or 4 equal slabs, slabs = 8 the graded start (four
    slabs of T/8, T/8, T/4, T/2)."""
    if K <= 0:
        return [0, 0]
    b = list(range(0, K, T)) + [K]
    if slabs == 8:
        if K >= T and T % 8 == 0 and T // 8 >= 16:
            b = [0, T // 8, T // 4, T // 2] + b[1:]
    elif slabs > 1 and K >= T and T % slabs == 0 and T // slabs >= 16:
        b = [i * (T // slabs) for i in range(slabs)] + b[1:]
    return b


def grids(M, N, K, T, slabs=1):
    c = lambda a: -(-a // T)
    return c(M), c(N), len(kbounds(K, T, slabs)) - 1


def check_plan(rows, stats, M, N, K, T, a_remote, b_remote, c_remote, beta_zero, pool_blocks, nq, slabs=1):
    Mg, Ng, Kg = grids(M, N, K, T, slabs)
    gemms = [r for r in rows if r["kind"] == GEMM]
    # every subkernel fired exactly once
    assert sorted((g["mi"], g["ni"], g["ki"]) for g in gemms) == sorted(itertools.product(range(Mg), range(Ng), range(Kg)))
    assert stats[5] == Mg * Ng * Kg
    chain = {}
    for idx, r in enumerate(rows):
        for w in r["waits"]:
            assert 0 <= w < idx, "dependencies point backwards only"
            assert rows[w]["stream"] != r["stream"], "same-stream order needs no event"
        if r["kind"] == GEMM:
            c = chain.setdefault((r["mi"], r["ni"]), [])
            # first K-step of a C tile: beta' = 0 into the accumulator (remote C) or the caller's beta (resident C)
            if not c:
                assert r["beta_mode"] == (BETA_ZERO if c_remote else BETA_USER)
            else:
                assert r["beta_mode"] == BETA_ONE
                assert r["stream"] == c[0]["stream"], "a C tile's K-chain stays on one exec queue"
                assert r["block"] == c[0]["block"]
            c.append(r)
            assert EXEC0 <= r["stream"] < EXEC0 + nq
            assert (r["a_block"] >= 0) == bool(a_remote) and (r["b_block"] >= 0) == bool(b_remote)
            assert (r["block"] >= 0) == bool(c_remote)
        if r["kind"] in (FETCH_A, FETCH_B, FETCH_C):
            assert r["stream"] == H2D and 0 <= r["block"] < pool_blocks
        if r["kind"] == WRITEBACK:
            assert r["stream"] == D2H
    assert all(len(c) == Kg for c in chain.values())
    n_wb = sum(r["kind"] == WRITEBACK for r in rows)
    n_red = sum(r["kind"] == REDUCE for r in rows)
    assert n_wb == (Mg * Ng if c_remote else 0)
    assert n_red == (Mg * Ng if (c_remote and not beta_zero) else 0)
    assert stats[3] == n_red
    assert stats[0] <= pool_blocks


def replay(rows, M, N, K, T, alpha, beta, A, B, C, pool_blocks, slabs=1):
    """Execute the plan sequentially in plan order with numpy tiles; checks along the way that every block is read
    only while it holds the tile the command expects (i.e. eviction never clobbers live data in plan order)."""
    kb = kbounds(K, T, slabs)
    sl = lambda i, D: slice(kb[i], kb[i + 1]) if D is K_AXIS else slice(i * T, min((i + 1) * T, D))
    blocks = [None] * pool_blocks
    out = C.copy()
    for r in rows:
        k = r["kind"]
        if k == FETCH_A:
            blocks[r["block"]] = ("A", r["mi"], r["ki"], A[sl(r["mi"], M), sl(r["ki"], K_AXIS)].copy())
        elif k == FETCH_B:
            blocks[r["block"]] = ("B", r["ki"], r["ni"], B[sl(r["ki"], K_AXIS), sl(r["ni"], N)].copy())
        elif k == FETCH_C:
            src = C[sl(r["mi"], M), sl(r["ni"], N)]
            if r.get("rows", 0) > 0:
                # a row strip of the caller's tile into those rows of the block
                if blocks[r["block"]] is None or blocks[r["block"]][:3] != ("S", r["mi"], r["ni"]):
                    blocks[r["block"]] = ("S", r["mi"], r["ni"], np.full(src.shape, np.nan))
                rs = slice(r["row0"], r["row0"] + r["rows"])
                blocks[r["block"]][3][rs] = src[rs]
            else:
                blocks[r["block"]] = ("S", r["mi"], r["ni"], src.copy())
        elif k == GEMM:
            if r["a_block"] >= 0:
                tag, i, j, a = blocks[r["a_block"]]
                assert (tag, i, j) == ("A", r["mi"], r["ki"])
            else:
                a = A[sl(r["mi"], M), sl(r["ki"], K_AXIS)]
            if r["b_block"] >= 0:
                tag, i, j, b = blocks[r["b_block"]]
                assert (tag, i, j) == ("B", r["ki"], r["ni"])
            else:
                b = B[sl(r["ki"], K_AXIS), sl(r["ni"], N)]
            if r.get("rows", 0) > 0:
                # a row strip of the tile (order ids of 640000 and above): those rows of the accumulator only
                assert r["block"] >= 0 and 0 <= r["row0"] and r["row0"] + r["rows"] <= a.shape[0]
                rs = slice(r["row0"], r["row0"] + r["rows"])
                prod = alpha * (a[rs] @ b)
                if blocks[r["block"]] is None or blocks[r["block"]][:3] != ("ACC", r["mi"], r["ni"]):
                    blocks[r["block"]] = ("ACC", r["mi"], r["ni"], np.full((a.shape[0], b.shape[1]), np.nan))
                acc = blocks[r["block"]][3]
                acc[rs] = prod if r["beta_mode"] == BETA_ZERO else acc[rs] + prod
                continue
            prod = alpha * (a @ b)
            if r["block"] >= 0:
                if r["beta_mode"] == BETA_ZERO:
                    blocks[r["block"]] = ("ACC", r["mi"], r["ni"], prod)
                else:
                    tag, i, j, acc = blocks[r["block"]]
                    assert (tag, i, j) == ("ACC", r["mi"], r["ni"]) and r["beta_mode"] == BETA_ONE
                    blocks[r["block"]] = ("ACC", i, j, acc + prod)
            else:
                tgt = out[sl(r["mi"], M), sl(r["ni"], N)]
                tgt[...] = prod + (beta if r["beta_mode"] == BETA_USER else 1.0) * tgt
        elif k == REDUCE:
            tag, i, j, acc = blocks[r["block"]]
            stag, si, sj, src = blocks[r["a_block"]]
            assert (tag, i, j) == ("ACC", r["mi"], r["ni"]) and (stag, si, sj) == ("S", r["mi"], r["ni"])
            if r.get("rows", 0) > 0:
                rs = slice(r["row0"], r["row0"] + r["rows"])
                acc[rs] = beta * src[rs] + acc[rs]
            else:
                blocks[r["block"]] = ("ACC", i, j, beta * src + acc)
        elif k == WRITEBACK:
            tag, i, j, acc = blocks[r["block"]]
            assert (tag, i, j) == ("ACC", r["mi"], r["ni"])
            if r.get("rows", 0) > 0:
                rs = slice(r["row0"], r["row0"] + r["rows"])
                out[sl(r["mi"], M), sl(r["ni"], N)][rs] = acc[rs]
            else:
                out[sl(r["mi"], M), sl(r["ni"], N)] = acc
    return out


def check_async_safety(rows):
    """Every data hazard on a pool block is ordered by stream order plus the recorded waits (transitively): a reader
    runs after the command that produced what it reads, and a command that overwrites a block runs after every
    earlier reader and writer of that block.  Commands on a row strip of a C tile touch those rows of the accumulator
    block only; hazards are between commands whose rows overlap.  Happens-before sets are bit masks."""
    whole = (0, 1 << 30)
    span = lambda r: (r["row0"], r["row0"] + r["rows"]) if r.get("rows", 0) > 0 else whole
    overlap = lambda a, b: a[0] < b[1] and b[0] < a[1]
    before = [0] * len(rows)
    last_on_stream = {}
    last_write = {}   # block -> [(rows, command that last wrote them)]
    users = {}        # block -> [(rows, command that read them since)]
    for i, r in enumerate(rows):
        deps = 0
        if r["stream"] in last_on_stream:
            j = last_on_stream[r["stream"]]
            deps |= before[j] | (1 << j)
        for w in r["waits"]:
            deps |= before[w] | (1 << w)
        before[i] = deps
        last_on_stream[r["stream"]] = i
        k = r["kind"]
        reads, writes = [], []
        if k in (FETCH_A, FETCH_B, FETCH_C):
            writes = [(r["block"], span(r))]
        elif k == GEMM:
            reads = [(x, whole) for x in (r["a_block"], r["b_block"]) if x >= 0]
            if r["block"] >= 0:
                (writes if r["beta_mode"] == BETA_ZERO else reads).append((r["block"], span(r)))
                if r["beta_mode"] != BETA_ZERO:
                    writes.append((r["block"], span(r)))
        elif k == REDUCE:
            reads = [(r["block"], span(r)), (r["a_block"], span(r))]
            writes = [(r["block"], span(r))]
        elif k == WRITEBACK:
            reads = [(r["block"], span(r))]
        for blk, sp in reads:
            ws = [w for wsp, w in last_write.get(blk, []) if overlap(wsp, sp)]
            assert ws, "cmd %d reads block %d that nothing wrote" % (i, blk)
            for w in ws:
                assert w == i or (deps >> w) & 1, "cmd %d reads block %d before its writer %d is known to be done" % (i, blk, w)
        for blk, sp in writes:
            for usp, u in users.get(blk, []) + last_write.get(blk, []):
                if overlap(usp, sp):
                    assert u == i or (deps >> u) & 1, "block %d overwritten by cmd %d before cmd %d is known to be done" % (blk, i, u)
        for blk, sp in reads:
            users.setdefault(blk, []).append((sp, i))
        for blk, sp in writes:
            # (what the new rows cover completely is superseded; a tile-wide entry stays beside a strip's)
            inside = lambda e: sp[0] <= e[0][0] and e[0][1] <= sp[1]
            last_write[blk] = [e for e in last_write.get(blk, []) if not inside(e)] + [(sp, i)]
            users[blk] = [e for e in users.get(blk, []) if not inside(e)]


ORDERS = [10000, 0, 1, 3, 10002, 10004, 20002, 30001, 50000, 60002, 102, 201, 202, 10201, 10999]


@pytest.mark.parametrize("order", ORDERS)
@pytest.mark.parametrize("locs", [(1, 1, 1), (1, 1, 0), (0, 1, 1), (1, 0, 0), (0, 0, 1)])
@pytest.mark.parametrize("beta_zero", [0, 1])
def test_plan_invariants_and_replay(pkg, order, locs, beta_zero):
    M, N, K, T = 90, 70, 110, 32
    a_r, b_r, c_r = locs
    rows, stats = pkg.plan_rows(M, N, K, T, a_r, b_r, c_r, beta_zero, 8, 2, 0, order)
    full = 1 + 3 * 4 + 4 * 3 + 2 * 3 * 3
    check_plan(rows, stats, M, N, K, T, a_r, b_r, c_r, beta_zero, full, 2)
    # everything fits: each remote tile is fetched exactly once, nothing is evicted
    assert stats[1] == (3 * 4 if a_r else 0) and stats[2] == (4 * 3 if b_r else 0) and stats[4] == 0
    rng = np.random.default_rng(order + 7 * beta_zero)
    A = rng.integers(-5, 6, (M, K)).astype(np.float64)
    B = rng.integers(-5, 6, (K, N)).astype(np.float64)
    C = rng.integers(-5, 6, (M, N)).astype(np.float64)
    alpha, beta = 2.0, (0.0 if beta_zero else 3.0)
    got = replay(rows, M, N, K, T, alpha, beta, A, B, C, full)
    assert np.array_equal(got, alpha * (A @ B) + beta * C)
    check_async_safety(rows)


@pytest.mark.parametrize("pool", [3, 4, 7, 12])
@pytest.mark.parametrize("beta_zero", [0, 1])
def test_plan_with_eviction(pkg, pool, beta_zero):
    """A pool smaller than the working set: tiles are re-fetched, nothing live is clobbered, a writer of a recycled
    block waits for every earlier user of that block."""
    M, N, K, T = 100, 100, 100, 32
    rows, stats = pkg.plan_rows(M, N, K, T, 1, 1, 1, beta_zero, 8, 2, pool, 10000)
    check_plan(rows, stats, M, N, K, T, 1, 1, 1, beta_zero, pool, 2)
    assert stats[4] > 0 and stats[1] + stats[2] > 2 * 16
    rng = np.random.default_rng(pool)
    A = rng.integers(-5, 6, (M, K)).astype(np.float64)
    B = rng.integers(-5, 6, (K, N)).astype(np.float64)
    C = rng.integers(-5, 6, (M, N)).astype(np.float64)
    beta = 0.0 if beta_zero else -2.0
    assert np.array_equal(replay(rows, M, N, K, T, 1.0, beta, A, B, C, pool), A @ B + beta * C)
    check_async_safety(rows)


def test_plan_too_small_pool_is_an_error(pkg):
    with pytest.raises(pkg.ParaliaError, match="< 3 blocks"):
        pkg.plan_rows(100, 100, 100, 32, 1, 1, 1, 0, 8, 2, 2, 10000)
    # k-outer order keeps every C accumulator open: it cannot run in 5 blocks, the reference order can
    with pytest.raises(pkg.ParaliaError, match="too small"):
        pkg.plan_rows(100, 100, 100, 32, 1, 1, 1, 0, 8, 2, 5, 4)
    pkg.plan_rows(100, 100, 100, 32, 1, 1, 1, 0, 8, 2, 5, 10000)


def test_reference_order_is_index_order(pkg):
    rows, _ = pkg.plan_rows(64, 96, 128, 32, 1, 1, 1, 1, 8, 2, 0, 10000)
    got = [(r["mi"], r["ni"], r["ki"]) for r in rows if r["kind"] == GEMM]
    assert got == list(itertools.product(range(2), range(3), range(4)))  # mi*Ng*Kg + ni*Kg + ki (dgemm.cpp:139-142)


def test_panel_starts_in_growing_squares(pkg):
    """First k-step of a panel order: after n fetched tiles the subkernels that can run must grow like a square, not
    one per fetch.  8 x 8 x 8 tiles, panel of 5 column tiles (order 5): the subkernels launched before the i-th fetch
    of the first k-step."""
    rows, _ = pkg.plan_rows(16384, 16384, 16384, 2048, 1, 1, 1, 1, 8, 2, 0, 5)
    first = [(r["mi"], r["ni"]) for r in rows if r["kind"] == GEMM and r["ki"] == 0][:40]
    assert first[:9] == [(0, 0), (0, 1), (1, 0), (1, 1), (0, 2), (1, 2), (2, 0), (2, 1), (2, 2)]
    assert sorted(first) == sorted(itertools.product(range(8), range(5)))     # the whole 8 x 5 panel, once each
    fetches_before = []
    n_fetch = 0
    for r in rows:
        if r["kind"] in (0, 1):
            n_fetch += 1
        elif r["kind"] == GEMM and r["ki"] == 0 and r["ni"] < 5:
            fetches_before.append(n_fetch)
    # 2 tiles -> 1 subkernel, 4 -> 4, 6 -> 9, 8 -> 16, 10 -> 25 (5 x 5), then one fetched A tile per 5 subkernels
    assert [fetches_before[i] for i in (0, 3, 8, 15, 24, 29, 39)] == [2, 4, 6, 8, 10, 11, 13]
    # every later k-step walks the panel the same way, and since the K chains were dealt to the two exec queues in that
    # order, consecutive subkernels of a step sit on different queues (column by column, column 0 of this panel would be
    # eight subkernels on one queue while the other waits for the next column's B tile)
    for ki in range(1, 8):
        step = [r for r in rows if r["kind"] == GEMM and r["ki"] == ki and r["ni"] < 5]
        assert [(r["mi"], r["ni"]) for r in step] == first
        assert all(a["stream"] != b["stream"] for a, b in zip(step, step[1:]))


def test_pipeline_simulation(pkg, L):
    import ctypes as C
    busy = (C.c_double * 3)()
    picked = C.c_int()
    # 16384^3, T = 2048, tile costs 0.24 ms compute / 0.6 ms each way: compute-bound overall (123 ms of kernels,
    # 77 ms of H2D, 38 ms of D2H); a good order hides nearly all transfers, the reference index order cannot hide
    # the fetch of a whole K-chain per C tile at the start, pure k-outer leaves every write-back to the end.
    args = (16384, 16384, 16384, 2048, 1, 1, 1, 1, 8, 2, 0)
    st = (0.24e-3, 0.0, 0.6e-3 / (2048 * 2048 * 8), 0.0, 0.6e-3 / (2048 * 2048 * 8), 0.02e-3, 1.0, 1.0)
    best = L.PARALiA_gemm_plan_simulate(*args, -1, *st, C.byref(picked), busy)
    # a thin start (order id 160000 * s + ...: first k tile in 2^s slabs) multiplies the same flops in more launches,
    # every slab priced at 2 us on top of its share of the tile time
    slabs = 1 << (picked.value // 160000)
    assert slabs in (1, 2, 4, 8)
    # (slabs of 1024 and deeper cost 2 us, shallower ones in inverse proportion to their depth; 8 = the graded start:
    # T/8, T/8, T/4, T/2 of a 2048-tile)
    extra = {1: 0.0, 2: 64 * 2 * 2e-6, 4: 64 * 4 * 4e-6, 8: 64 * (8e-6 + 8e-6 + 4e-6 + 2e-6)}[slabs]
    assert abs(busy[1] - (512 * 0.24e-3 + extra)) < 1e-9
    assert abs(busy[0] - 128 * 0.6e-3) < 1e-9 and abs(busy[2] - 64 * 0.6e-3) < 1e-9
    unsplit = L.PARALiA_gemm_plan_simulate(*args, picked.value % 160000, *st, None, None)
    assert best <= unsplit                              # and is only taken when the simulated call gets shorter
    assert best >= busy[1] and best < busy[1] * 1.04
    ref_order = L.PARALiA_gemm_plan_simulate(*args, 10000, *st, None, None)
    k_outer = L.PARALiA_gemm_plan_simulate(*args, 8, *st, None, None)
    assert best <= ref_order and best <= k_outer
    assert k_outer > busy[1] + 0.5 * busy[2]          # write-backs pile up behind the last K step
    serial = busy[0] + busy[1] + busy[2]
    assert best < 0.6 * serial
    # transfer-bound case (40000 x 40000 x 2048, beta != 0): the H2D stream is the critical resource
    args5 = (40000, 40000, 2048, 2048, 1, 1, 1, 0, 8, 2, 0)
    t5 = L.PARALiA_gemm_plan_simulate(*args5, -1, *st, C.byref(picked), busy)
    assert busy[0] > busy[1] and t5 >= busy[0] and t5 < busy[0] * 1.05


def test_pipeline_simulation_link_contention(pkg, L):
    """Copies in opposite directions slow each other by the link model's sl factors.  Checked on cases whose answer
    is known without running the simulator's own arithmetic: (1) sl = 1 changes nothing; (2) a D2H slowdown alone can
    only lengthen the makespan and the D2H busy time, never the H2D busy time; (3) in the transfer-bound 40000 x 40000
    x 2048 case the D2H stream is busy nearly the whole time, so the H2D busy time must land between the undisturbed
    time and sl times it, and close to sl times it."""
    import ctypes as C
    busy0, busy1 = (C.c_double * 3)(), (C.c_double * 3)()
    tb = 0.6e-3 / (2048 * 2048 * 8)
    args5 = (40000, 40000, 2048, 2048, 1, 1, 1, 0, 8, 2, 0)
    base = (0.24e-3, 0.0, tb, 0.0, tb, 0.02e-3)
    t0 = L.PARALiA_gemm_plan_simulate(*args5, 10000, *base, 1.0, 1.0, None, busy0)
    t_d = L.PARALiA_gemm_plan_simulate(*args5, 10000, *base, 1.0, 1.3, None, busy1)
    assert t_d >= t0 and busy1[2] > busy0[2] * 1.05 and abs(busy1[0] - busy0[0]) < 1e-12
    t_h = L.PARALiA_gemm_plan_simulate(*args5, 10000, *base, 1.2, 1.0, None, busy1)
    assert busy0[0] * 1.12 < busy1[0] <= busy0[0] * 1.2 + 1e-9
    assert t_h >= busy1[0] and t_h > t0 * 1.1
    assert abs(busy1[2] - busy0[2]) < 1e-12
    # compute-bound 16384^3 with beta = 0: transfers hide behind the kernels either way, the makespan barely moves
    args3 = (16384, 16384, 16384, 2048, 1, 1, 1, 1, 8, 2, 0)
    a = L.PARALiA_gemm_plan_simulate(*args3, 4, *base, 1.0, 1.0, None, None)
    b = L.PARALiA_gemm_plan_simulate(*args3, 4, *base, 1.2, 1.2, None, None)
    assert a <= b < a * 1.03


@pytest.mark.parametrize("threads", [1, 3, 8])
@pytest.mark.parametrize("rows,cols,ld", [(1, 1, 1), (37, 91, 50), (2048, 300, 2048), (1000, 1, 4000), (5, 4000, 9)])
def test_host_copy2d_gather_and_scatter(L, threads, rows, cols, ld):
    """The threaded strided host copy behind the pageable-operand path: gather a sub-matrix into a dense tile and
    scatter it back; bytes outside the sub-matrix must stay untouched."""
    import numpy as np
    rng = np.random.default_rng(rows * cols + threads)
    src = rng.random(ld * cols)
    dense = np.full(rows * cols, -1.0)
    assert L.PARALiA_host_copy2d(dense.ctypes.data, rows * 8, src.ctypes.data, ld * 8, rows * 8, cols, threads) == 0
    assert np.array_equal(dense.reshape(cols, rows), src.reshape(cols, ld)[:, :rows])
    back = np.full(ld * cols, -2.0)
    assert L.PARALiA_host_copy2d(back.ctypes.data, ld * 8, dense.ctypes.data, rows * 8, rows * 8, cols, threads) == 0
    assert np.array_equal(back.reshape(cols, ld)[:, :rows], src.reshape(cols, ld)[:, :rows])
    assert np.all(back.reshape(cols, ld)[:, rows:] == -2.0)
    assert L.PARALiA_host_copy2d(back.ctypes.data, rows * 8 - 1, dense.ctypes.data, rows * 8, rows * 8, cols, threads) != 0


@pytest.mark.parametrize("seed", range(60))
def test_random_plans_are_safe_and_correct(pkg, seed):
    """Random shapes (ragged tiles, K = 0 and T larger than a dimension included), operand placements, order families
    and pool sizes from the minimum to the full working set: every plan that builds must keep all invariants, replay to
    the exact result and order every hazard; a plan that does not fit must say so."""
    rng = np.random.default_rng(1000 + seed)
    M, N = (int(x) for x in rng.integers(1, 200, 2))
    K = int(rng.integers(0, 200))
    T = int(rng.choice([16, 24, 32, 50, 64, 128, 256]))
    a_r, b_r, c_r = (int(x) for x in rng.integers(0, 2, 3))
    beta_zero = int(rng.integers(0, 2))
    nq = int(rng.integers(1, 5))
    Mg, Ng, Kg = grids(M, N, K, T)
    full = 1 + Mg * Kg + Kg * Ng + 2 * Mg * Ng
    pool = int(rng.choice([0, 3, 4, 5, max(3, full // 3), max(3, full // 2), full]))
    orient, w = int(rng.integers(0, 2)), int(rng.integers(0, max(Mg, Ng) + 2))
    order = orient * 10000 + w + (20000 if w > 0 and rng.integers(0, 2) else 0) + (40000 if rng.integers(0, 2) else 0)
    if seed % 5 == 4:   # a block order: rows * 100 + columns, plain or with the other eviction policy
        order = orient * 10000 + int(rng.integers(1, Mg + 2)) * 100 + int(rng.integers(1, Ng + 2)) + (40000 if rng.integers(0, 2) else 0)
    A = rng.integers(-4, 5, (M, K)).astype(np.float64)
    B = rng.integers(-4, 5, (K, N)).astype(np.float64)
    C = rng.integers(-4, 5, (M, N)).astype(np.float64)
    alpha, beta = 2.0, (0.0 if beta_zero else -3.0)
    try:
        rows, stats = pkg.plan_rows(M, N, K, T, a_r, b_r, c_r, beta_zero, 8, nq, pool, order)
    except pkg.ParaliaError as e:
        assert (a_r or b_r or c_r) and pool and pool < full and ("too small" in str(e) or "< 3 blocks" in str(e))
        return
    eff_pool = pool if pool else full
    check_plan(rows, stats, M, N, K, T, a_r, b_r, c_r, beta_zero, eff_pool, nq)
    assert np.array_equal(replay(rows, M, N, K, T, alpha, beta, A, B, C, eff_pool), alpha * (A @ B) + beta * C)
    check_async_safety(rows)


def expand_merged(rows):
    """A plan with merged K chains (order ids of 80000 and above) rewritten as the equivalent plan with one GEMM row per
    k tile, so that the checks above apply unchanged: the k tiles of a launch sit in consecutive blocks of its panels,
    the launch's waits guard its first k-step, later k-steps follow on the same stream, and whoever waited for the
    launch waits for its last k-step."""
    out, new_index = [], {}
    for i, r in enumerate(rows):
        if r["kind"] == GEMM and r["kn"] > 1:
            for s in range(r["kn"]):
                e = dict(r, ki=r["ki"] + s, kn=1, waits=list(r["waits"]) if s == 0 else [],
                         a_block=r["a_block"] + s if r["a_block"] >= 0 else -1, b_block=r["b_block"] + s if r["b_block"] >= 0 else -1,
                         beta_mode=r["beta_mode"] if s == 0 else BETA_ONE)
                out.append(e)
        else:
            out.append(dict(r, waits=list(r["waits"])))
        new_index[i] = len(out) - 1
    for e in out:
        e["waits"] = [new_index[w] for w in e["waits"]]
    return out


@pytest.mark.parametrize("order", [80000, 80001, 80002, 90000, 90002])
@pytest.mark.parametrize("locs", [(1, 1, 1), (1, 1, 0), (0, 1, 1), (1, 0, 0)])
@pytest.mark.parametrize("beta_zero", [0, 1])
def test_merged_chain_plans(pkg, order, locs, beta_zero):
    """Merged K chains: fewer GEMM launches than subkernels, every (mi, ni, ki) still covered exactly once, the tiles of
    A and B in their fixed panel blocks (A(mi, ki) in block mi * Kg + ki, B(ki, ni) behind them in ni * Kg + ki), each
    fetched once, and the expanded plan keeps every invariant, replays exactly and orders every hazard."""
    M, N, K, T = 90, 70, 110, 32
    a_r, b_r, c_r = locs
    Mg, Ng, Kg = grids(M, N, K, T)
    rows, stats = pkg.plan_rows(M, N, K, T, a_r, b_r, c_r, beta_zero, 8, 2, 0, order)
    gemms = [r for r in rows if r["kind"] == GEMM]
    assert sum(g["kn"] for g in gemms) == Mg * Ng * Kg and len(gemms) < Mg * Ng * Kg
    assert any(g["kn"] == Kg for g in gemms)                  # the tile-by-tile part of the order runs whole chains
    a_first = 0
    b_first = Mg * Kg if a_r else 0
    for r in rows:
        if r["kind"] == FETCH_A:
            assert r["block"] == a_first + r["mi"] * Kg + r["ki"]
        if r["kind"] == FETCH_B:
            assert r["block"] == b_first + r["ni"] * Kg + r["ki"]
    full = 1 + Mg * Kg + Kg * Ng + 2 * Mg * Ng
    flat = expand_merged(rows)
    check_plan(flat, stats, M, N, K, T, a_r, b_r, c_r, beta_zero, full, 2)
    assert stats[1] == (Mg * Kg if a_r else 0) and stats[2] == (Kg * Ng if b_r else 0) and stats[4] == 0
    rng = np.random.default_rng(order + beta_zero)
    A = rng.integers(-5, 6, (M, K)).astype(np.float64)
    B = rng.integers(-5, 6, (K, N)).astype(np.float64)
    C = rng.integers(-5, 6, (M, N)).astype(np.float64)
    alpha, beta = 2.0, (0.0 if beta_zero else 3.0)
    assert np.array_equal(replay(flat, M, N, K, T, alpha, beta, A, B, C, full), alpha * (A @ B) + beta * C)
    check_async_safety(flat)


def test_merged_chains_need_the_whole_working_set_and_pay_only_with_a_saving(pkg, L):
    import ctypes as C
    with pytest.raises(pkg.ParaliaError, match="panel layout"):
        pkg.plan_rows(100, 100, 100, 32, 1, 1, 1, 0, 8, 2, 12, 80000)     # 4 x 4 tiles of A and of B do not fit 12 blocks
    # simulator: the same order with and without merging costs the same when a merged launch saves nothing ...
    args = (4096, 4096, 4096, 512, 1, 1, 0, 0, 4, 2, 0)
    st = (1e-3, 1e-5, 2e-11, 1e-5, 2e-11, 1e-5, 1.0, 1.0)
    picked, busy = C.c_int(), (C.c_double * 3)()
    plain = L.PARALiA_gemm_plan_simulate(*args, 2, *st, C.byref(picked), busy)
    merged = L.PARALiA_gemm_plan_simulate(*args, 80002, *st, C.byref(picked), busy)
    assert plain > 0 and abs(merged - plain) <= 1e-9 * plain
    # ... and the search offers merged orders only to a kernel with such a saving (none through this entry point)
    best = L.PARALiA_gemm_plan_simulate(*args, -1, *st, C.byref(picked), busy)
    assert picked.value % 160000 < 80000 and best <= plain


@pytest.mark.parametrize("order", [160000, 160002, 170001, 320000, 320003, 330002, 240002, 410001, 180002, 480000, 490002, 560001, 480203])
@pytest.mark.parametrize("locs", [(1, 1, 1), (1, 1, 0), (0, 1, 1), (1, 0, 0)])
@pytest.mark.parametrize("beta_zero", [0, 1])
def test_thin_start_plans(pkg, order, locs, beta_zero):
    """Order ids of 160000 * s and above: the first k tile is cut into slabs (s = 1: two, s = 2: four equal ones, s = 3:
    the graded start of T/8, T/8, T/4, T/2), each a k tile of its own (fetched into its own block, multiplied by its
    own launch, beta' = 0 on a C tile's first slab only).  Every subkernel of the finer k grid fires once, every tile
    is fetched once, and the plan -- with merged K chains expanded -- keeps the invariants, replays to the exact result
    on integers and orders every hazard.  K = 110 with T = 32: 4 k tiles become 5 (two slabs of 16); four slabs of 8
    are too thin, so ids of 320000 and above are refused here, as they are when K < T; the graded start needs T = 128
    (slabs of 16, 16, 32, 64)."""
    M, N, K, T = 90, 70, 110, 32
    a_r, b_r, c_r = locs
    slabs = 1 << (order // 160000)
    if slabs >= 4:
        with pytest.raises(pkg.ParaliaError, match="thin start"):
            pkg.plan_rows(M, N, K, T, a_r, b_r, c_r, beta_zero, 8, 2, 0, order)
        T = 64                                                   # 2 k tiles become 5: slabs of 16, 16, 16, 16 and 46
    if slabs == 8:
        with pytest.raises(pkg.ParaliaError, match="thin start"):
            pkg.plan_rows(M, N, K, T, a_r, b_r, c_r, beta_zero, 8, 2, 0, order)     # an eighth of 64 is too thin
        M, N, K, T = 300, 200, 310, 128                          # 3 k tiles become 6: 16, 16, 32, 64, 128 and 54
    Mg, Ng, Kg = grids(M, N, K, T, slabs)
    assert Kg == -(-K // T) + min(slabs, 4) - 1
    if slabs == 8:
        assert kbounds(K, T, 8) == [0, 16, 32, 64, 128, 256, 310]
    rows, stats = pkg.plan_rows(M, N, K, T, a_r, b_r, c_r, beta_zero, 8, 2, 0, order)
    flat = expand_merged(rows)
    full = 1 + Mg * Kg + Kg * Ng + 2 * Mg * Ng
    check_plan(flat, stats, M, N, K, T, a_r, b_r, c_r, beta_zero, full, 2, slabs)
    assert stats[1] == (Mg * Kg if a_r else 0) and stats[2] == (Kg * Ng if b_r else 0) and stats[4] == 0
    rng = np.random.default_rng(order + beta_zero)
    A = rng.integers(-5, 6, (M, K)).astype(np.float64)
    B = rng.integers(-5, 6, (K, N)).astype(np.float64)
    C = rng.integers(-5, 6, (M, N)).astype(np.float64)
    alpha, beta = 2.0, (0.0 if beta_zero else 3.0)
    assert np.array_equal(replay(flat, M, N, K, T, alpha, beta, A, B, C, full, slabs), alpha * (A @ B) + beta * C)
    check_async_safety(flat)
    with pytest.raises(pkg.ParaliaError, match="thin start"):
        pkg.plan_rows(M, N, 20, 32, a_r, b_r, c_r, beta_zero, 8, 2, 0, order)     # K < T: nothing to cut


@pytest.mark.parametrize("order", [640000, 650002, 720000, 720002, 730001, 880001, 720203, 660003, 700001])
@pytest.mark.parametrize("locs", [(1, 1, 1), (0, 1, 1), (1, 0, 1)])
@pytest.mark.parametrize("beta_zero", [1, 0])
def test_strip_end_plans(pkg, order, locs, beta_zero):
    """Order ids of 640000 and above: the last launch of the call -- the last k-step of the C tile the order completes
    last, or that tile's whole merged K chain -- is made in row strips, each a launch of its own over the same k range
    that says how many ways it splits K, and what follows on the tile comes strip by strip as well: with beta != 0 the
    fetch of the caller's C and the lazy reduce, then the write-back.  Everything before that launch is the plan of
    the id without the flag; the strips cover the tile's rows once; the plan replays to the exact result and orders
    every hazard, strips against strips by their rows (with a pool smaller than the working set too: 660003, 700001).
    Where the flag does not apply (C on the device, a last tile under 512 rows) the plan is that of the plain id."""
    a_r, b_r, c_r = locs
    M, N, K, T = 1300, 1100, 1200, 512                              # last tile 276 x 76: nothing to cut
    pool = 14 if order % 80000 >= 20000 else 0
    plain_id = order - 640000
    assert pkg.plan_rows(M, N, K, T, a_r, b_r, c_r, beta_zero, 8, 2, pool, order)[0] == pkg.plan_rows(M, N, K, T, a_r, b_r, c_r, beta_zero, 8, 2, pool, plain_id)[0]
    M = 1536                                                        # last tile 512 x 76 -> strips of 256 rows
    if order % 10000 == 203:
        M, N = 2048, 1636                                           # the block order ends on tile (3, 3): 512 x 100
    assert pkg.plan_rows(M, N, K, T, a_r, b_r, 0, beta_zero, 8, 2, pool, order)[0] == pkg.plan_rows(M, N, K, T, a_r, b_r, 0, beta_zero, 8, 2, pool, plain_id)[0]
    slabs = 1 << (plain_id // 160000)
    merged = plain_id % 160000 >= 80000
    Mg, Ng, Kg = grids(M, N, K, T, slabs)
    plain, _ = pkg.plan_rows(M, N, K, T, a_r, b_r, c_r, beta_zero, 8, 2, pool, plain_id)
    rows, stats = pkg.plan_rows(M, N, K, T, a_r, b_r, c_r, beta_zero, 8, 2, pool, order)
    at = max(i for i, r in enumerate(plain) if r["kind"] == GEMM)
    last = plain[at]
    assert last["kn"] == (Kg if merged else 1) and last["ki"] + last["kn"] == Kg
    assert [r["kind"] for r in plain[at:]] == ([GEMM, WRITEBACK] if beta_zero else [GEMM, FETCH_C, REDUCE, WRITEBACK])
    assert rows[:at] == plain[:at] and all(r["rows"] == 0 and r["splits"] == 0 for r in rows[:at])
    tail = rows[at:]
    tm, tn = M - last["mi"] * T, N - last["ni"] * T
    assert tm == 512 and len(tail) == (4 if beta_zero else 8)       # two strips of 256 rows
    kinds = [GEMM, WRITEBACK] if beta_zero else [GEMM, FETCH_C, REDUCE, WRITEBACK]
    assert [r["kind"] for r in tail] == [k for k in kinds for _ in range(2)]
    launch_k = K if merged else K - (K // T) * T
    for i, r in enumerate(tail):
        assert (r["mi"], r["ni"]) == (last["mi"], last["ni"]) and (r["row0"], r["rows"]) == (256 * (i % 2), 256)
        if r["kind"] == GEMM:
            assert (r["ki"], r["kn"], r["beta_mode"], r["stream"], r["block"]) == (last["ki"], last["kn"], last["beta_mode"], last["stream"], last["block"])
            assert (r["a_block"], r["b_block"]) == (last["a_block"], last["b_block"])
            assert r["splits"] == max(1, min(-(-512 // (2 * -(-tn // 128))), launch_k // 512)) == (2 if merged else 1)
        elif r["kind"] == WRITEBACK:
            assert r["block"] == last["block"] and r["waits"] == [at + (4 if not beta_zero else 0) + i % 2]
        elif r["kind"] == REDUCE:
            assert r["block"] == last["block"] and r["stream"] == last["stream"] and at + 2 + i % 2 in r["waits"]
    flat = expand_merged(rows)
    full = pool if pool else 1 + Mg * Kg + Kg * Ng + 2 * Mg * Ng
    rng = np.random.default_rng(order)
    A = rng.integers(-5, 6, (M, K)).astype(np.float64)
    B = rng.integers(-5, 6, (K, N)).astype(np.float64)
    C = rng.integers(-5, 6, (M, N)).astype(np.float64)
    beta = 0.0 if beta_zero else 3.0
    assert np.array_equal(replay(flat, M, N, K, T, 2.0, beta, A, B, C, full, slabs), 2.0 * (A @ B) + beta * C)
    check_async_safety(flat)


def test_block_orders(pkg):
    """w = rows * 100 + columns: that block of C tiles is the k-outer panel (walked in growing squares in every k-step),
    the rest follows tile by tile with the K chain innermost -- for orient 0 the other rows of the block's columns, then
    the other columns."""
    M = N = K = 4 * 64
    rows, _ = pkg.plan_rows(M, N, K, 64, 1, 1, 1, 1, 8, 2, 0, 302)
    g = [(r["mi"], r["ni"], r["ki"]) for r in rows if r["kind"] == GEMM]
    block = [(0, 0), (0, 1), (1, 0), (1, 1), (2, 0), (2, 1)]
    assert g[:24] == [(mi, ni, ki) for ki in range(4) for (mi, ni) in block]
    assert g[24:32] == [(3, ni, ki) for ni in range(2) for ki in range(4)]
    assert g[32:] == [(mi, ni, ki) for ni in (2, 3) for mi in range(4) for ki in range(4)]
    rows, _ = pkg.plan_rows(M, N, K, 64, 1, 1, 1, 1, 8, 2, 0, 10302)
    g = [(r["mi"], r["ni"], r["ki"]) for r in rows if r["kind"] == GEMM]
    assert g[24:48] == [(mi, ni, ki) for ni in (2, 3) for mi in range(3) for ki in range(4)]
    assert g[48:] == [(3, ni, ki) for ni in range(4) for ki in range(4)]
    # the first C tile goes back after three k-steps of the block (3 + 2 tiles each) and two tiles of the last one; a
    # panel over all rows needs 4 + 2 tiles per k-step
    def fetched_before_first_writeback(plan_rows):
        n_fetch = 0
        for r in plan_rows:
            if r["kind"] in (FETCH_A, FETCH_B):
                n_fetch += 1
            if r["kind"] == WRITEBACK:
                break
        return n_fetch
    assert fetched_before_first_writeback(rows) == 3 * 5 + 2
    assert fetched_before_first_writeback(pkg.plan_rows(M, N, K, 64, 1, 1, 1, 1, 8, 2, 0, 2)[0]) == 3 * 6 + 2
    # a block larger than the grid is the grid; repeated panels have no block form; zero columns is no order
    rows, stats = pkg.plan_rows(M, N, K, 64, 1, 1, 1, 1, 8, 2, 0, 9999)
    check_plan(rows, stats, M, N, K, 64, 1, 1, 1, 1, 1 << 20, 2)
    for order in (20302, 300):
        with pytest.raises(pkg.ParaliaError, match="unknown order id"):
            pkg.plan_rows(M, N, K, 64, 1, 1, 1, 1, 8, 2, 0, order)
    # merged chains and thin start combine with it
    for order in (80302, 160302, 240302):
        rows, stats = pkg.plan_rows(M, N, K, 64, 1, 1, 1, 1, 8, 2, 0, order)
        assert stats[5] == 4 * 4 * (4 if order < 160000 else 5)


def test_whole_grid_panel_on_grids_of_a_hundred_tiles_and_more(pkg, L):
    """Panel widths live below 100 in the order id (100 and above encode blocks), and 99 stands for the whole grid.  On a
    128 x 128 grid of C tiles (M = N = 32768 at T = 256) the whole-grid panel is still a candidate and is planned as one:
    the first k-step fires all 128 x 128 subkernels before the second starts."""
    import ctypes as C
    T, g = 256, 128
    M = N = g * T
    rows, stats = pkg.plan_rows(M, N, 2 * T, T, 1, 1, 0, 0, 8, 2, 0, 99)
    gem = [(r["mi"], r["ni"], r["ki"]) for r in rows if r["kind"] == GEMM]
    assert len(gem) == g * g * 2 and all(ki == 0 for (_, _, ki) in gem[:g * g]) and all(ki == 1 for (_, _, ki) in gem[g * g:])
    assert sorted((mi, ni) for (mi, ni, _) in gem[:g * g]) == [(mi, ni) for mi in range(g) for ni in range(g)]
    rows10, _ = pkg.plan_rows(M, N, 2 * T, T, 1, 1, 0, 0, 8, 2, 0, 10099)
    assert [(r["mi"], r["ni"], r["ki"]) for r in rows10 if r["kind"] == GEMM][:g * g] == gem[:g * g]
    # width 98 is a panel of 98 columns, not the grid
    rows98, _ = pkg.plan_rows(M, N, 2 * T, T, 1, 1, 0, 0, 8, 2, 0, 98)
    gem98 = [(r["mi"], r["ni"], r["ki"]) for r in rows98 if r["kind"] == GEMM]
    assert all(ni < 98 for (_, ni, _) in gem98[:2 * g * 98]) and gem98[2 * g * 98][1] == 98
    # the order search still simulates the whole-grid panel on such a grid: pinned to it, the simulator accepts the id
    picked = C.c_int(-1)
    busy = (C.c_double * 3)()
    t = L.PARALiA_gemm_plan_simulate(M, N, 2 * T, T, 1, 1, 0, 0, 8, 2, 0, 99, 1e-5, 1e-6, 1e-11, 1e-6, 1e-11, 1e-6, 1.0, 1.0, C.byref(picked), busy)
    assert t > 0 and picked.value == 99


def test_unknown_order_ids_are_refused(pkg):
    for order in (1280000, 1440001, -5):
        with pytest.raises(pkg.ParaliaError, match="unknown order id"):
            pkg.plan_rows(256, 256, 256, 64, 1, 1, 1, 0, 8, 2, 0, order)
