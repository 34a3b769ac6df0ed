"""Row-block plan layout, checked on the CPU: the host-side builder
(mps_rowblock_layout_build) against a Python walk that decodes the streams the
way the kernel does (rows_advanced marks, per-step tables, shared-row slots),
and against the structure the layout promises.  No GPU, no oracle needed: the
product of the walk is compared with a dense fp64 product."""
import numpy as np
import pytest

from tests.gpu_util import random_csr

G, WAVES, WSLOTS, WIN = 16, 16, 16, 4


def dealt_len(n, g):
    return n // G + (1 if g < n % G else 0)


def rounds_for(n):
    """rounds (two windows per lane-group each) a wavefront needs for n windows dealt to its 16 lane-groups"""
    return (n // G + (1 if n % G else 0) + 1) // 2


def walk_layout(pkg, lay, X, n):
    """Y = A @ X from the layout alone, in the order the kernel uses; also returns the
    original nonzero indices seen (from the source arrays)."""
    C = pkg._cabi
    i = lay.info
    T, H, NB = i.rowblock_steps, i.rowblock_table_rows, i.rowblock_blocks
    hot_bits, cold_bits = i.hot_mark_shift, i.mark_shift
    brow = lay.array(C.MPS_PLAN_ARRAY_RB_BLOCK_ROW, np.int32)
    hot_cols = lay.array(C.MPS_PLAN_ARRAY_RB_HOT_COLS, np.int32).reshape(T, H)
    table_base = lay.array(C.MPS_PLAN_ARRAY_RB_TABLE_BASE, np.int32)
    assert table_base.size == (NB if i.rowblock_local_tables else 0)
    meta = lay.array(C.MPS_PLAN_ARRAY_RB_META, np.int32).reshape(NB, T, WSLOTS, 4)
    base = lay.array(C.MPS_PLAN_ARRAY_RB_WAVE_BASE, np.int64).reshape(NB, WSLOTS, 2)
    streams = [lay.array(C.MPS_PLAN_ARRAY_RB_HOT, np.uint32).reshape(-1, 2),
               lay.array(C.MPS_PLAN_ARRAY_RB_COLD, np.uint32).reshape(-1, 2)]
    srcs = [lay.array(C.MPS_PLAN_ARRAY_RB_HOT_SRC, np.int32), lay.array(C.MPS_PLAN_ARRAY_RB_COLD_SRC, np.int32)]
    bits = [hot_bits, cold_bits]
    Y = np.zeros((n, X.shape[1]), dtype=np.float64)
    seen = []
    assert brow[0] == 0 and brow[-1] == n and (np.diff(brow) > 0).all()
    assert (np.diff(brow) <= i.rowblock_acc_rows).all()
    for b in range(NB):
        row0, nr = int(brow[b]), int(brow[b + 1] - brow[b])
        acc = np.zeros((i.rowblock_acc_rows, X.shape[1]))
        cur = base[b].copy()
        for t in range(T):
            if i.rowblock_local_tables:  # the block's own H consecutive rows of X (zeros beyond its end)
                cols = int(table_base[b]) + t * H + np.arange(H)
                table = np.where((cols < n)[:, None], X[np.minimum(cols, n - 1)], 0.0)
            else:
                table = np.where(hot_cols[t][:, None] >= 0, X[np.maximum(hot_cols[t], 0)], 0.0)
            firsts = meta[b, t, :WAVES, 2]
            assert (np.diff(firsts) >= 0).all(), "first rows of the wavefronts' runs must not decrease"
            slots = np.zeros((WAVES, X.shape[1]))
            for w in range(WAVES):
                first_row = int(firsts[w])
                for k in range(2):
                    nk = int(meta[b, t, w, k])  # windows of this wavefront's run
                    for g in range(G):
                        row, part, any_entry = first_row, np.zeros(X.shape[1]), False
                        for jw in range(dealt_len(nk, g)):
                            # round jw // 2; lane (g, e) holds entry e of the group's two windows side by side
                            slot0 = (int(cur[w, k]) + jw // 2) * (G * WIN * 2) + g * WIN * 2 + jw % 2
                            adv = int(streams[k][slot0, 0]) >> bits[k]
                            if adv:
                                (slots[w] if row == first_row else acc[row]).__iadd__(part)
                                part = np.zeros(X.shape[1])
                                row += adv
                            assert 0 <= row < nr
                            real = 0
                            for e in range(WIN):
                                word, vbits = int(streams[k][slot0 + 2 * e, 0]), streams[k][slot0 + 2 * e, 1]
                                val = float(np.array([vbits], dtype=np.uint32).view(np.float32)[0])
                                idx = word & ((1 << bits[k]) - 1)
                                assert e == 0 or (word >> bits[k]) == 0, "only a window's first entry advances rows"
                                x = table[idx] if k == 0 else X[idx]
                                if k == 0:
                                    assert hot_cols[t, idx] >= 0 or (i.rowblock_local_tables and table_base[b] + t * H + idx < n)
                                src = int(srcs[k][slot0 + 2 * e])
                                if src >= 0:
                                    assert real == e, "a window's nonzeros come first, padding after them"
                                    real += 1
                                    seen.append(src)
                                else:
                                    assert val == 0.0, "padding carries the value 0"
                                part = part + val * x
                            assert real >= 1
                            any_entry = True
                        if any_entry:
                            (slots[w] if row == first_row else acc[row]).__iadd__(part)
                    cur[w, k] += rounds_for(nk)
            for w in range(WAVES):
                acc[int(firsts[w])] += slots[w]
        for k in range(2):
            for w in range(WAVES - 1):
                assert cur[w, k] == base[b, w + 1, k], "a wavefront's streams end where the next one's begin"
        Y[row0:row0 + nr] = acc[:nr]
    return Y, np.array(seen, dtype=np.int64)


CASES = [
    # n, max_deg, hubs, steps, table_rows, block_rows, blocks_per_round
    (2000, 3, ((5, 1500),), 2, 16, 1000, 2),  # sparse: hot windows more than 31 rows apart
    (300, 40, ((5, 280), (150, 300)), 3, 16, 64, 4),
    (97, 12, (), 2, 8, 0, 2),
    (513, 60, ((0, 500), (512, 400)), 5, 32, 40, 8),
    (64, 64, ((10, 64),), 1, 64, 0, 1),
    (200, 5, (), 4, 4, 16, 256),
]


@pytest.mark.parametrize("case", CASES)
def test_layout_walk_reproduces_the_product(pkg, case):
    n, max_deg, hubs, steps, table_rows, block_rows, per_round = case
    rng = np.random.default_rng(hash(case) % (2 ** 32))
    rp, ci = random_csr(rng, n, max_deg, p_empty=0.25, hub_rows=hubs)
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, 16)) * 2 - 1).astype(np.float32)
    lay = pkg.spmm.RowBlockLayout(rp, ci, val, K=16, steps=steps, table_rows=table_rows, block_rows=block_rows,
                                  blocks_per_round=per_round)
    assert lay.info.rowblock_steps == steps and lay.info.rowblock_table_rows == table_rows
    Y, seen = walk_layout(pkg, lay, X.astype(np.float64), n)
    # every nonzero exactly once
    assert np.array_equal(np.sort(seen), np.arange(ci.size))
    A = np.zeros((n, n))
    rows = np.repeat(np.arange(n), np.diff(rp))
    A[rows, ci] = val
    ref = A @ X.astype(np.float64)
    assert np.allclose(Y, ref, rtol=1e-12, atol=1e-12)
    # padding slots hold no source
    C = pkg._cabi
    for which in (C.MPS_PLAN_ARRAY_RB_HOT_SRC, C.MPS_PLAN_ARRAY_RB_COLD_SRC):
        src = lay.array(which, np.int32)
        assert ((src >= 0).sum() + 0) <= ci.size
    hot_src = lay.array(C.MPS_PLAN_ARRAY_RB_HOT_SRC, np.int32)
    assert (hot_src >= 0).sum() == lay.info.hot_nnz
    # the packed form of the hot stream, what the device reads: the same entries, 12 bytes per lane and round
    # {value A, value B, half A | half B << 16}; a half is the table slot and, above bit 11, a 5-bit piece of the
    # window's rows_advanced (entry 0: the low piece, entry 1: the high one)
    hot = lay.array(C.MPS_PLAN_ARRAY_RB_HOT, np.uint32).reshape(-1, 2)
    packed = lay.array(C.MPS_PLAN_ARRAY_RB_HOT_PACKED, np.uint32).reshape(-1, 3)  # one row per (round, lane)
    bits = lay.info.hot_mark_shift
    assert bits <= 11 and packed.shape[0] * 2 == hot.shape[0]
    assert np.array_equal(packed[:, 0], hot[0::2, 1]) and np.array_equal(packed[:, 1], hot[1::2, 1])
    slot = (hot[:, 0] & ((1 << bits) - 1)).reshape(-1, 64, 2)   # [round][lane][A / B]
    adv = (hot[:, 0] >> bits).reshape(-1, 16, 4, 2)             # [round][group][entry][A / B]
    assert adv.max(initial=0) < 1024 and not adv[:, :, 1:, :].any()
    piece = np.zeros_like(adv)
    piece[:, :, 0, :] = adv[:, :, 0, :] & 31
    piece[:, :, 1, :] = adv[:, :, 0, :] >> 5
    half = slot | (piece.reshape(-1, 64, 2) << 11)
    assert np.array_equal(packed[:, 2].reshape(-1, 64), half[:, :, 0] | (half[:, :, 1] << 16))
    # the packed form of the cold stream, where it fits: the same 12 bytes; a half is the column counted from the
    # first column of the step's range and, above index_bits, the piece of rows_advanced that belongs to the entry
    # (entry e: bits [e p, (e + 1) p), p = 16 - index_bits)
    ib = lay.info.rowblock_cold_index_bits
    cpk = lay.array(C.MPS_PLAN_ARRAY_RB_COLD_PACKED, np.uint32).reshape(-1, 3)
    if ib == 0:
        assert cpk.size == 0
        return
    pb = 16 - ib
    cold = lay.array(C.MPS_PLAN_ARRAY_RB_COLD, np.uint32).reshape(-1, 2)
    cold_begin = lay.array(C.MPS_PLAN_ARRAY_RB_COLD_BEGIN, np.int32)
    cbits = lay.info.mark_shift
    assert 12 <= ib <= 15 and cpk.shape[0] * 2 == cold.shape[0] and cold_begin.size == lay.info.rowblock_steps + 1
    assert np.array_equal(cpk[:, 0], cold[0::2, 1]) and np.array_equal(cpk[:, 1], cold[1::2, 1])
    half = np.stack([cpk[:, 2] & 0xffff, cpk[:, 2] >> 16], axis=1).reshape(-1, 16, 4, 2)  # [round][group][entry][A / B]
    rel, piece = half & ((1 << ib) - 1), half >> ib
    adv_packed = sum(piece[:, :, e, :].astype(np.int64) << (pb * e) for e in range(4))       # [round][group][A / B]
    col = (cold[:, 0] & ((1 << cbits) - 1)).reshape(-1, 16, 4, 2).astype(np.int64)
    adv = (cold[:, 0] >> cbits).reshape(-1, 16, 4, 2)[:, :, 0, :]
    # rounds in stream order belong to (block, wavefront, step): walk them the way the builder laid them out
    meta = lay.array(C.MPS_PLAN_ARRAY_RB_META, np.int32).reshape(lay.info.rowblock_blocks, lay.info.rowblock_steps, WSLOTS, 4)
    base = lay.array(C.MPS_PLAN_ARRAY_RB_WAVE_BASE, np.int64).reshape(lay.info.rowblock_blocks, WSLOTS, 2)
    for b in range(lay.info.rowblock_blocks):
        for w in range(WAVES):
            r = int(base[b, w, 1])
            for t in range(lay.info.rowblock_steps):
                nk = int(meta[b, t, w, 1])
                for q in range(rounds_for(nk)):
                    for g in range(G):
                        for which in range(2):
                            if 2 * q + which < dealt_len(nk, g):
                                assert np.array_equal(rel[r, g, :, which] + cold_begin[t], col[r, g, :, which])
                                assert adv_packed[r, g, which] == adv[r, g, which]
                            else:
                                assert not half[r, g, :, which].any()
                    r += 1


def greedy_cuts(win, slack_div=8):
    """The runs of one (block, step), restated: win[row, kind] windows in row order (a row's hot ones, then its cold
    ones); run w begins within a run's length / slack_div of w E / 16, where the rounds of run w - 1 get the least
    padding; among equals the nearest to w E / 16, then the first."""
    kind = np.repeat(np.tile([0, 1], win.shape[0]), win.ravel())
    E = kind.size
    before = [np.concatenate([[0], np.cumsum(kind == k)]) for k in range(2)]
    pad = lambda x: rounds_for(int(x)) * 32 - int(x)
    slack = E // WAVES // slack_div
    cuts = [0]
    for w in range(1, WAVES):
        equal = w * E // WAVES
        if E == 0:
            cuts.append(0)
            continue
        lo, hi = max(cuts[-1], equal - slack), min(equal + slack, E - 1)
        cuts.append(min(range(lo, hi + 1), key=lambda q: (pad(before[0][q] - before[0][cuts[-1]]) +
                                                           pad(before[1][q] - before[1][cuts[-1]]), abs(q - equal), q)))
    cuts.append(E)
    return [[int(before[k][cuts[w + 1]] - before[k][cuts[w]]) for k in range(2)] for w in range(WAVES)], cuts, E


def test_runs_are_cut_where_their_last_rounds_fill(pkg):
    C = pkg._cabi
    rng = np.random.default_rng(77)
    n, T, H = 1500, 6, 32
    rp, ci = random_csr(rng, n, 300, p_empty=0.05, hub_rows=((3, 1400), (900, 1200)))
    val = rng.random(ci.size).astype(np.float32)
    lay = pkg.spmm.RowBlockLayout(rp, ci, val, K=16, steps=T, table_rows=H, block_rows=0, blocks_per_round=2, keep_sources=False)
    i = lay.info
    NB = i.rowblock_blocks
    brow = lay.array(C.MPS_PLAN_ARRAY_RB_BLOCK_ROW, np.int32)
    hot_cols = lay.array(C.MPS_PLAN_ARRAY_RB_HOT_COLS, np.int32).reshape(T, H)
    cold_begin = lay.array(C.MPS_PLAN_ARRAY_RB_COLD_BEGIN, np.int32)
    meta = lay.array(C.MPS_PLAN_ARRAY_RB_META, np.int32).reshape(NB, T, WSLOTS, 4)
    col_step, col_hot = np.zeros(n, dtype=np.int64), np.zeros(n, dtype=bool)
    for t in range(T):
        col_step[cold_begin[t]:cold_begin[t + 1]] = t
    for t in range(T):
        c = hot_cols[t][hot_cols[t] >= 0]
        col_step[c], col_hot[c] = t, True
    moved, slots, slots_equal, windows = 0, 0, 0, 0
    for b in range(NB):
        r0, r1 = int(brow[b]), int(brow[b + 1])
        rows = np.repeat(np.arange(r1 - r0), np.diff(rp[r0:r1 + 1]))
        cols = ci[rp[r0]:rp[r1]]
        key = (col_step[cols] * (r1 - r0) + rows) * 2 + (~col_hot[cols])
        win = (np.bincount(key, minlength=T * (r1 - r0) * 2).reshape(T, r1 - r0, 2) + 3) // 4
        for t in range(T):
            want, cuts, E = greedy_cuts(win[t])
            assert meta[b, t, :WAVES, :2].tolist() == want, (b, t)
            assert all(abs(cuts[w] - w * E // WAVES) <= E // WAVES // 8 for w in range(WAVES + 1))
            moved += sum(cuts[w] != w * E // WAVES for w in range(WAVES))
            equal, _, _ = greedy_cuts(win[t], slack_div=10 ** 9)  # no slack: the cuts at w E / 16
            slots += sum(rounds_for(x) * 32 for run in want for x in run)
            slots_equal += sum(rounds_for(x) * 32 for run in equal for x in run)
            windows += E
    assert moved > NB * T * 8           # most cuts found a better place
    assert slots - windows < 0.5 * (slots_equal - windows)   # and the last rounds hold less than half the padding


def test_hot_columns_are_the_busiest_and_dealt_round_robin(pkg):
    rng = np.random.default_rng(3)
    n = 400
    rp, ci = random_csr(rng, n, 80, p_empty=0.1, hub_rows=((7, 390),))
    val = np.ones(ci.size, dtype=np.float32)
    T, H = 4, 20
    lay = pkg.spmm.RowBlockLayout(rp, ci, val, steps=T, table_rows=H, blocks_per_round=4)
    hot_cols = lay.array(pkg._cabi.MPS_PLAN_ARRAY_RB_HOT_COLS, np.int32).reshape(T, H)
    deg = np.bincount(ci, minlength=n)
    order = sorted(range(n), key=lambda c: (-deg[c], c))[:T * H]
    for k, c in enumerate(order):
        assert hot_cols[k % T, k // T] == c
    assert lay.info.hot_nnz == deg[order].sum()


def test_blocks_balance_nonzeros(pkg):
    rng = np.random.default_rng(5)
    n = 4000
    rp, ci = random_csr(rng, n, 30, p_empty=0.3, hub_rows=((100, 3000), (2000, 2500), (3999, 1000)))
    val = np.ones(ci.size, dtype=np.float32)
    lay = pkg.spmm.RowBlockLayout(rp, ci, val, steps=2, table_rows=64, blocks_per_round=16)
    brow = lay.array(pkg._cabi.MPS_PLAN_ARRAY_RB_BLOCK_ROW, np.int32)
    assert brow.size - 1 == 16
    per_block = rp[brow[1:]] - rp[brow[:-1]]
    # no block holds more than the average plus the longest row
    assert per_block.max() <= ci.size / 16 + np.diff(rp).max()


def test_more_rounds_of_blocks_where_one_round_is_unequal(pkg):
    """16 x 1,024 rows at 16 blocks per round: one round means blocks of exactly 1,024 rows, and the first of them
    would hold seven eighths of the nonzeros.  The builder adds rounds until no block is more than half above its
    share (two rounds: 15 blocks are full of short rows, which leaves 17 for the long ones, 1.6 times the share)."""
    rng = np.random.default_rng(6)
    n = 16 * 1024
    deg = np.where(np.arange(n) < 1024, 200, 2)
    rp = np.zeros(n + 1, dtype=np.int32)
    rp[1:] = np.cumsum(deg)
    ci = np.concatenate([np.sort(rng.choice(n, size=d, replace=False)) for d in deg]).astype(np.int32)
    val = np.ones(ci.size, dtype=np.float32)
    lay = pkg.spmm.RowBlockLayout(rp, ci, val, steps=1, table_rows=64, blocks_per_round=16, keep_sources=False)
    brow = lay.array(pkg._cabi.MPS_PLAN_ARRAY_RB_BLOCK_ROW, np.int32)
    per_block = rp[brow[1:]] - rp[brow[:-1]]
    assert 32 < brow.size - 1 <= 48 and per_block.max() <= 1.5 * ci.size / 48
    assert (np.diff(brow) <= 1024).all()
    # rows that one round does hold in equal blocks stay in one round
    deg2 = np.full(n // 2, 20)
    rp2 = np.zeros(n // 2 + 1, dtype=np.int32)
    rp2[1:] = np.cumsum(deg2)
    ci2 = np.concatenate([np.sort(rng.choice(n // 2, size=20, replace=False)) for _ in deg2]).astype(np.int32)
    lay2 = pkg.spmm.RowBlockLayout(rp2, ci2, np.ones(ci2.size, dtype=np.float32), steps=1, table_rows=64, blocks_per_round=16,
                                   keep_sources=False)
    assert lay2.info.rowblock_blocks == 16


@pytest.mark.parametrize("spec,steps,why", [
    ("er:n=120000,deg=60", 3, "7.7 MB of X, columns used evenly: 3 MiB a step"),
    ("chunglu:n=120000,nnz=7200000,gamma=2.1,dmax=4000", 2, "7.7 MB of X, skewed columns: 5 MiB a step"),
    ("er:n=120000,deg=20", 1, "9,400 nonzeros per block: a second step would leave fewer than 5,000 each"),
    ("chunglu:n=30000,nnz=16000000,gamma=2.1,dmax=6000", 2, "X fits one step, but a block has 62,500 nonzeros: a second table"),
    ("er:n=190000,deg=190", 4, "141,000 nonzeros per block ask for 5 tables, but a table serves 0.9 % of them: 12.2 MB of X at 3 MiB a step"),
])
def test_steps_follow_the_size_of_x_the_work_and_the_skew(pkg, spec, steps, why):
    rp, ci, _ = pkg.graphs.generate(spec, seed=4)
    lay = pkg.spmm.RowBlockLayout(rp, ci, np.ones(ci.size, dtype=np.float32), keep_sources=False)
    assert lay.info.rowblock_steps == steps, why


@pytest.mark.parametrize("spec,steps,table_rows,block_rows,per_round,share,want_steps", [
    ("blockdiag:blocks=40,min=50,max=200,deg=5", 0, 0, 0, 4, 0.95, 1),    # a table covers a block's components
    ("blockdiag:blocks=40,min=50,max=200,deg=5", 1, 64, 100, 4, 0.2, 1),  # one table narrower than a component: many cold entries
    ("blockdiag:blocks=40,min=50,max=200,deg=5", 0, 64, 100, 4, 0.8, 5),  # as many tables of 64 rows as the blocks' column spans need
    ("blockdiag:blocks=40,min=50,max=200,deg=5", 3, 32, 50, 4, 0.3, 3),   # three tables of 32 rows, cold columns on either side
    ("er:n=300,deg=6", 0, 0, 0, 2, 1.0, 1),                                # fewer columns than table rows: everything is hot
    ("er:n=300,deg=6", 0, 20, 16, 2, 0.4, 8),                              # columns all over: 8 tables at most
])
def test_local_tables_walk_reproduces_the_product(pkg, spec, steps, table_rows, block_rows, per_round, share, want_steps):
    """MPS_PLAN_LOCAL_TABLES: block b's table of step t holds the columns base[b] + t H .. base[b] + (t + 1) H - 1
    (base[b]: the window of T H columns with the most of the block's nonzeros), RB_HOT_COLS is unused; the walk over
    the streams gives the product."""
    rp, ci, _ = pkg.graphs.generate(spec, seed=3)
    n = rp.size - 1
    rng = np.random.default_rng(12)
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, 16)) * 2 - 1).astype(np.float64)
    lay = pkg.spmm.RowBlockLayout(rp, ci, val, steps=steps, table_rows=table_rows, block_rows=block_rows,
                                  blocks_per_round=per_round, local_tables=True)
    i = lay.info
    assert i.rowblock_local_tables == 1 and i.rowblock_steps == want_steps
    assert (lay.array(pkg._cabi.MPS_PLAN_ARRAY_RB_HOT_COLS, np.int32) == -1).all()
    base = lay.array(pkg._cabi.MPS_PLAN_ARRAY_RB_TABLE_BASE, np.int32)
    brow = lay.array(pkg._cabi.MPS_PLAN_ARRAY_RB_BLOCK_ROW, np.int32)
    width = i.rowblock_steps * i.rowblock_table_rows
    assert (base >= 0).all() and (base <= max(0, n - width)).all()
    # hot_nnz counts the nonzeros whose column lies in their block's window
    blk = np.repeat(np.arange(brow.size - 1), rp[brow[1:]] - rp[brow[:-1]])
    inside = (ci >= base[blk]) & (ci < base[blk] + width)
    assert i.hot_nnz == int(inside.sum()) and i.hot_nnz >= share * ci.size - 1e-9
    Y, seen = walk_layout(pkg, lay, X, n)
    assert np.array_equal(np.sort(seen), np.arange(ci.size))
    A = np.zeros((n, n))
    A[np.repeat(np.arange(n), np.diff(rp)), ci] = val
    assert np.allclose(Y, A @ X, rtol=1e-12, atol=1e-12)
    # without the flag the same matrix gets global tables
    assert pkg.spmm.RowBlockLayout(rp, ci, val, blocks_per_round=per_round).info.rowblock_local_tables == 0


def test_rejects_what_it_is_not_built_for(pkg):
    rp = np.array([0, 1, 2], dtype=np.int32)
    ci = np.array([0, 1], dtype=np.int32)
    val = np.ones(2, dtype=np.float32)
    with pytest.raises(pkg._cabi.MpsError) as e:
        pkg.spmm.RowBlockLayout(rp, ci, val, K=32)
    assert e.value.status == pkg._cabi.MPS_ERR_UNSUPPORTED
    with pytest.raises(pkg._cabi.MpsError):
        pkg.spmm.RowBlockLayout(rp, ci, val, K=16, table_rows=100000)
