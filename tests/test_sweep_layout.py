"""The layout of a sweep plan (mps_sweep_layout_build, host only): walked here the way the kernel walks it, and
checked for the rules the kernel relies on."""
import numpy as np
import pytest
import scipy.sparse as sps

from tests.gpu_util import random_csr

WAVES, ROUND_INSTR = 16, 8


def swizzle(v, G):
    return v ^ (((v >> 2) ^ (v >> 4) ^ (v >> 6)) & (G - 1))


def walk(pkg, lay, n, K, X, elem_bytes):
    """Y as the kernel forms it (fp64 sums), plus the rule checks."""
    C = pkg._cabi
    i = lay.info
    L, tiles, cb, acc_rows, NP = i.sweep_lanes, i.sweep_tiles, i.sweep_col_bits, i.sweep_acc_rows, i.sweep_panels
    together = i.sweep_together
    assert together in (1, 2)
    gpw = 64 // L
    G = max(1, 256 // (16 * L))
    assert (tiles - 1) * L * 16 < K * elem_bytes <= tiles * L * 16 and L == (4 if K * elem_bytes <= 64 else 8)
    panel_ptr = lay.array(C.MPS_PLAN_ARRAY_SW_PANEL_PTR, np.int32)
    rows = lay.array(C.MPS_PLAN_ARRAY_SW_ROWS, np.int32)
    piece_ptr = lay.array(C.MPS_PLAN_ARRAY_SW_PIECE_PTR, np.int32)
    meta = lay.array(C.MPS_PLAN_ARRAY_SW_WAVE_META, np.int32).reshape(NP * WAVES, 2)
    prounds = lay.array(C.MPS_PLAN_ARRAY_SW_PANEL_ROUNDS, np.int32)
    stream = lay.array(C.MPS_PLAN_ARRAY_SW_STREAM, np.uint32)
    src = lay.array(C.MPS_PLAN_ARRAY_SW_SRC, np.int32)
    split_row = lay.array(C.MPS_PLAN_ARRAY_SW_SPLIT_ROW, np.int32)
    split_ptr = lay.array(C.MPS_PLAN_ARRAY_SW_SPLIT_PTR, np.int32)
    assert stream.size == 2 * i.sweep_slots and src.size == i.sweep_slots
    assert i.sweep_rounds * gpw * ROUND_INSTR == i.sweep_slots
    assert rows.size == i.sweep_listed_rows == panel_ptr[-1]
    st = stream.reshape(-1, gpw * 4, 2, 2)  # [round][lane-group * 4 + lane of quad][window A / B][word, value]
    sr = src.reshape(-1, gpw * 4, 2)
    n_partial = split_ptr[-1] if split_ptr.size else 0
    Y = np.full((n + n_partial, K), np.nan)
    seen = np.zeros(max(i.nnz, 1), dtype=np.int64)
    wave_entries = np.zeros(NP * WAVES, dtype=np.int64)
    for b in range(NP):
        acc = np.zeros((acc_rows + 1, K))
        owner = np.full(acc_rows + 1, -1)
        most = 0
        for w in range(WAVES):
            first, rounds = meta[b * WAVES + w]
            most = max(most, rounds)
            last_col = -1
            for r in range(first, first + rounds):
                rows_of = {}  # (window, lane of quad) -> accumulator rows of that instruction
                for t in range(ROUND_INSTR):
                    win, q = t // 4, t % 4
                    for g in range(gpw):
                        word, vb = st[r, g * 4 + q, win]
                        e = sr[r, g * 4 + q, win]
                        col, vr = int(word) & ((1 << cb) - 1), int(word) >> cb
                        v = float(np.array([vb], np.uint32).view(np.float32)[0])
                        if e < 0:
                            assert v == 0.0 and vr == acc_rows  # padding: nothing into a real accumulator row
                        else:
                            assert vr < acc_rows
                            assert owner[vr] in (-1, w), "an accumulator row belongs to one wavefront"
                            owner[vr] = w
                            rows_of.setdefault((win, q), []).append(vr)
                            seen[e] += 1
                            wave_entries[b * WAVES + w] += 1
                        acc[vr] += v * X[col]
                # what is added up at the same time never shares an accumulator row: the entries of one instruction,
                # or (together == 2) of entry q of both windows
                for q in range(4):
                    groups = [rows_of.get((0, q), []) + rows_of.get((1, q), [])] if together == 2 else \
                        [rows_of.get((0, q), []), rows_of.get((1, q), [])]
                    for rows_here in groups:
                        assert len(set(rows_here)) == len(rows_here), "two entries added up at the same time share an accumulator row"
        assert prounds[b] == most
        p0, p1 = panel_ptr[b], panel_ptr[b + 1]
        pp = piece_ptr[p0 + b:p1 + b + 1]
        assert pp[0] == 0 and (np.diff(pp) >= 0).all() and pp[-1] <= acc_rows
        for k in range(p0, p1):
            pieces = [swizzle(p, G) for p in range(pp[k - p0], pp[k - p0 + 1])]
            assert np.isnan(Y[rows[k]]).all(), "a row is written once"
            Y[rows[k]] = acc[pieces].sum(axis=0) if pieces else 0.0
    if i.nnz:
        assert (seen[:i.nnz] == 1).all(), "every nonzero sits in exactly one slot"
    out = Y[:n].copy()
    for k, r in enumerate(split_row):
        assert np.isnan(out[r]).all()
        out[r] = Y[n + split_ptr[k]:n + split_ptr[k + 1]].sum(axis=0)
    assert not np.isnan(out).any(), "every row is written"
    return out, wave_entries


CASES = [
    # n, max_deg, hubs, K, elem_bytes, piece, acc_rows, panels_per_round, together
    (300, 12, ((5, 280),), 16, 4, 0, 0, 4, 0),
    (97, 6, (), 32, 4, 4, 0, 2, 0),
    (513, 20, ((0, 500), (512, 400)), 64, 4, 8, 64, 3, 0),
    (200, 5, (), 16, 4, 2, 16, 8, 0),            # few accumulator rows per panel: several rounds of panels
    (257, 9, ((100, 257),), 64, 2, 0, 0, 4, 0),  # fp16: 128-byte rows, two accumulator planes
    (64, 3, (), 32, 2, 0, 0, 1, 0),              # fp16, 64-byte rows: rows dealt in pairs
    (1, 1, (), 16, 4, 0, 0, 2, 0),
    (300, 12, ((5, 280),), 16, 4, 0, 0, 4, 2),   # 64-byte rows with pairs of instructions
    (400, 9, ((100, 257),), 32, 4, 0, 0, 4, 1),  # 128-byte rows, one instruction at a time
    (150, 8, ((7, 140),), 12, 4, 0, 0, 2, 0),    # 48-byte rows: one tile of 4 lanes, one of them idle
    (220, 8, ((9, 200),), 41, 4, 0, 0, 2, 0),    # 164-byte rows: two tiles of 8 lanes
    (180, 8, ((3, 170),), 40, 2, 0, 0, 2, 0),    # fp16, 80-byte rows
]


@pytest.mark.parametrize("case", CASES)
def test_sweep_layout_walk(pkg, case):
    n, max_deg, hubs, K, eb, piece, acc_rows, per_round, together = case
    rng = np.random.default_rng(abs(hash(case)) % (2 ** 32))
    rp, ci = random_csr(rng, n, max_deg, p_empty=0.3, hub_rows=hubs)
    val = rng.random(ci.size).astype(np.float32)
    X = rng.random((n, K)) * 2 - 1
    lay = pkg.spmm.SweepLayout(rp, ci, val, K, elem_bytes=eb, piece=piece, acc_rows=acc_rows, panels_per_round=per_round,
                               together=together)
    assert lay.info.sweep_panels % per_round == 0
    assert lay.info.sweep_together == (together or (2 if lay.info.sweep_lanes == 4 else 1))
    Y, wave_entries = walk(pkg, lay, n, K, X, eb)
    ref = sps.csr_matrix((val.astype(np.float64), ci, rp), shape=(n, n)) @ X
    assert np.allclose(Y, ref, rtol=1e-12, atol=1e-12)


def test_sweep_layout_balance_and_split(pkg):
    # one row holds a third of the nonzeros: it is cut into sub-rows for different panels, and the panels end up even
    rng = np.random.default_rng(5)
    n = 16000
    rp, ci = random_csr(rng, n, 10, p_empty=0.2, hub_rows=((17, 15000),))
    val = rng.random(ci.size).astype(np.float32)
    lay = pkg.spmm.SweepLayout(rp, ci, val, 16, panels_per_round=8)
    i = lay.info
    assert i.sweep_split_rows == 1 and i.sweep_partial_rows >= 2
    X = rng.random((n, 16)) * 2 - 1
    Y, wave_entries = walk(pkg, lay, n, 16, X, 4)
    ref = sps.csr_matrix((val.astype(np.float64), ci, rp), shape=(n, n)) @ X
    assert np.allclose(Y, ref, rtol=1e-12, atol=1e-12)
    per_panel = wave_entries.reshape(i.sweep_panels, WAVES).sum(axis=1)
    assert per_panel.max() <= 1.1 * per_panel.mean() + 16
    # padding: the last round of every wavefront, and instructions that a wavefront with few rows cannot fill
    assert i.sweep_slots <= 1.25 * ci.size + i.sweep_panels * WAVES * (64 // i.sweep_lanes) * ROUND_INSTR


def test_sweep_layout_rejects_what_it_cannot_hold(pkg):
    rp = np.array([0, 1, 2], dtype=np.int32)
    ci = np.array([0, 1], dtype=np.int32)
    val = np.ones(2, dtype=np.float32)
    with pytest.raises(pkg._cabi.MpsError) as e:
        pkg.spmm.SweepLayout(rp, ci, val, 13, elem_bytes=2)  # rows of X of 26 bytes: they start between two dwords
    assert e.value.status == pkg._cabi.MPS_ERR_UNSUPPORTED
