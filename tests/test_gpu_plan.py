"""Plans (mps_plan_*): column-slab tiling, partition of the virtual rows and
sliced nonzero arrays, checked against numpy restatements of their layout; the
SpMM through a plan meets the same bar against the oracle's fp64 row loop."""
import numpy as np
import pytest
import torch

from gpu_util import check_fp16, check_fp32, make_csr, random_csr, to_dev

pytestmark = pytest.mark.gpu


def slab_major_reference(rp, ci, num_slabs, slab_cols):
    """(vrow_ptr, perm): virtual row s*n + r holds row r's nonzeros with
    s*slab_cols <= col < (s+1)*slab_cols, in their original order."""
    n = rp.size - 1
    rows = np.repeat(np.arange(n, dtype=np.int64), np.diff(rp))
    slab = np.minimum(ci.astype(np.int64) // slab_cols, num_slabs - 1)
    v = slab * n + rows
    perm = np.argsort(v, kind="stable")
    counts = np.bincount(v, minlength=num_slabs * n)
    vrp = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    return vrp, perm.astype(np.int32)


def hot_reference(rp, ci, num_slabs, slab_cols, hot_rows):
    """(hot_slot[n], hot_cols[num_slabs * hot_rows]): per slab the hot_rows
    columns with the most nonzeros (ties to the smaller id, unreferenced
    columns never), slots in ascending column order."""
    n = rp.size - 1
    deg = np.bincount(ci, minlength=n)
    hot_slot = np.full(n, -1, dtype=np.int64)
    hot_cols = np.full(num_slabs * hot_rows, -1, dtype=np.int32)
    for s in range(num_slabs):
        c0, c1 = min(s * slab_cols, n), min((s + 1) * slab_cols, n)
        cols = np.arange(c0, c1)
        order = cols[np.lexsort((cols, -deg[c0:c1]))][:hot_rows]
        order = np.sort(order[deg[order] > 0])
        hot_slot[order] = np.arange(order.size)
        hot_cols[s * hot_rows:s * hot_rows + order.size] = order
    return hot_slot, hot_cols


def segment_major_reference(rp, ci, num_slabs, slab_cols, hot_slot):
    """Like slab_major_reference with 2 * num_slabs segments: segment s holds
    the nonzeros of slab s in hot columns, segment num_slabs + s the others."""
    n = rp.size - 1
    rows = np.repeat(np.arange(n, dtype=np.int64), np.diff(rp))
    slab = np.minimum(ci.astype(np.int64) // slab_cols, num_slabs - 1)
    seg = np.where(hot_slot[ci] >= 0, slab, num_slabs + slab)
    v = seg * n + rows
    perm = np.argsort(v, kind="stable")
    counts = np.bincount(v, minlength=2 * num_slabs * n)
    vrp = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    return vrp, perm.astype(np.int32)


def segmented_partition_reference(orc, vrp, n, num_slabs, cost, hot_cost, G):
    """Every segment split on its own with the reference search and padded
    with empty partitions to whole wavefronts.  Returns (xs, ys, hot_partitions)."""
    xs, ys = [], []
    hot_parts = 0
    for g in range(2 * num_slabs):
        seg_rp = vrp[g * n:(g + 1) * n + 1].astype(np.int64)
        y0 = int(seg_rp[0])
        nnz_g = int(seg_rp[-1]) - y0
        total = n + 1 + nnz_g
        parts = max(1, (total - 1) // (hot_cost if g < num_slabs else cost))
        lx, ly = orc.partition_coords((seg_rp - y0).astype(np.int32), nnz_g, parts)
        padded = -(-parts // G) * G
        lx = np.concatenate([lx[:parts], np.full(padded - parts, n + 1)])
        ly = np.concatenate([ly[:parts], np.full(padded - parts, nnz_g)])
        xs.append(g * n + np.maximum(lx, 1))
        ys.append(y0 + ly)
        if g < num_slabs:
            hot_parts += padded
    xs.append([2 * num_slabs * n + 1])
    ys.append([int(vrp[-1])])
    return np.concatenate(xs).astype(np.int32), np.concatenate(ys).astype(np.int32), hot_parts


def check_plan_layout(pkg, orc, plan, rp, ci, val):
    c, i = pkg._cabi, plan.info
    n, nnz = rp.size - 1, ci.size
    if i.hot_rows > 0:
        hot_slot, hot_cols = hot_reference(rp, ci, i.num_slabs, i.slab_cols, i.hot_rows)
        # one piece (16 partitions) for each of the 16 wavefronts of 256 workgroups, within 64 .. 256 items
        hot_items = i.num_slabs * (n + 1) + int((hot_slot[ci] >= 0).sum())
        assert i.num_segments == 2 * i.num_slabs and i.hot_cost == max(i.cost, min(256, max(64, hot_items // 65536)))
        assert np.array_equal(plan.array(c.MPS_PLAN_ARRAY_HOT_COLS), hot_cols)
        assert i.hot_nnz == int((hot_slot[ci] >= 0).sum())
        vrp, perm = segment_major_reference(rp, ci, i.num_slabs, i.slab_cols, hot_slot)
        assert np.array_equal(plan.array(c.MPS_PLAN_ARRAY_VROW_PTR), vrp)
        xs, ys, hot_parts = segmented_partition_reference(orc, vrp, n, i.num_slabs, i.cost, i.hot_cost, i.threads_per_wave)
        assert i.num_partitions == xs.size - 1 and i.hot_waves * i.threads_per_wave == hot_parts
        want_cols = np.where(hot_slot[ci] >= 0, hot_slot[ci], ci)  # hot nonzeros carry their LDS slot
    else:
        assert i.num_segments == i.num_slabs and i.hot_waves == 0 and i.hot_nnz == 0
        vrp, perm = slab_major_reference(rp, ci, i.num_slabs, i.slab_cols)
        assert np.array_equal(plan.array(c.MPS_PLAN_ARRAY_VROW_PTR), vrp)
        # the partition of the virtual rows is the reference split (oracle restatement)
        assert i.num_partitions == orc.num_partitions(i.num_slabs * n, nnz, i.cost)
        xs, ys = orc.partition_coords(vrp, nnz, i.num_partitions)
        want_cols = ci
    assert np.array_equal(plan.array(c.MPS_PLAN_ARRAY_COORD_X), xs)
    assert np.array_equal(plan.array(c.MPS_PLAN_ARRAY_COORD_Y), ys)
    # slices: wave w, round r, group g, element j  <-  virtual nonzero ys[p] + 16 r + j
    G, W = i.threads_per_wave, i.num_waves
    cnt = np.diff(ys)
    rounds = np.zeros(W, dtype=np.int64)
    for w in range(W):
        seg = cnt[w * G:(w + 1) * G]
        rounds[w] = ((seg + 15) // 16).max() if seg.size else 0
    wave_off = np.concatenate([[0], np.cumsum(rounds)])
    assert np.array_equal(plan.array(c.MPS_PLAN_ARRAY_WAVE_OFF), wave_off)
    assert i.total_rounds == wave_off[-1] and i.slice_slots == wave_off[-1] * G * 16
    src = plan.array(c.MPS_PLAN_ARRAY_SLICE_SRC)
    cols = plan.array(c.MPS_PLAN_ARRAY_SLICE_COLS)
    vals = plan.array(c.MPS_PLAN_ARRAY_SLICE_VALS)
    want_src = np.full(src.size, -1, dtype=np.int64)
    for p in range(i.num_partitions):
        w, g = divmod(p, G)
        k = np.arange(cnt[p])
        slot = (wave_off[w] + k // 16) * (G * 16) + g * 16 + k % 16
        want_src[slot] = perm[ys[p] + k]
    assert np.array_equal(src, want_src)
    live = want_src >= 0
    assert live.sum() == nnz
    # column entries: column (or LDS slot) below the mark shift, above it the number of rows that end in front
    # of the nonzero inside its partition
    row_of = np.searchsorted(vrp, np.arange(nnz), side="right") - 1
    ends = np.diff(row_of, prepend=0)
    first = ys[:-1][cnt > 0]
    ends[first] = row_of[first] - (np.maximum(xs[:-1][cnt > 0], 1) - 1)
    slot_part = np.repeat(np.arange(W), (wave_off[1:] - wave_off[:-1]) * G * 16)  # wave of every slot
    shift = np.where(slot_part < i.hot_waves, i.hot_mark_shift, i.mark_shift)
    assert (i.hot_mark_shift > 0) == (i.hot_rows > 0)
    cols_u = cols.astype(np.int64) & 0xFFFFFFFF
    got_col = np.where(shift > 0, cols_u & ((1 << shift) - 1), cols_u)
    # plans with resident columns: one flag bit (gather with the streaming hint) between column and row ends
    flag_bits = 1 if i.resident_cols > 0 else 0
    got_ends = np.where(shift > 0, cols_u >> (shift + flag_bits), 0)
    if flag_bits:
        deg = np.bincount(ci, minlength=n)
        order = sorted(range(n), key=lambda col: (-deg[col], col))[:i.resident_cols]
        assert all(deg[col] > 0 for col in order) and i.resident_nnz == int(deg[order].sum())
        streamed = np.ones(n, dtype=np.int64)
        streamed[order] = 0
        assert np.array_equal(((cols_u >> shift) & 1)[live], streamed[want_cols[want_src[live]]])
    inv = np.empty(nnz, dtype=np.int64)
    inv[perm] = np.arange(nnz)  # original nonzero -> virtual position
    vpos = inv[want_src[live]]
    assert np.array_equal(got_col[live], want_cols[want_src[live]]) and (cols[~live] == 0).all()
    assert np.array_equal(got_ends[live], np.where(shift[live] > 0, ends[vpos], 0))
    assert np.array_equal(vals[live], val[want_src[live]]) and (vals[~live] == 0).all()


@pytest.mark.parametrize("tiling,slab_bytes,cost,tpw,hot",
                         [("off", 0, 16, 0, "auto"), ("force", 16384, 16, 0, "off"), ("force", 4096, 7, 3, "off"),
                          ("force", 1 << 20, 64, 16, "off"), ("force", 8192, 128, 1, "off"),
                          ("force", 16384, 16, 0, "force"), ("force", 4096, 7, 3, "force"), ("force", 8192, 128, 1, "auto"),
                          ("force", 8192, 128, 1, "force")])
def test_plan_layout_matches_numpy(pkg, orc, dev, tiling, slab_bytes, cost, tpw, hot):
    rng = np.random.default_rng(cost + slab_bytes)
    n = 500
    rp, ci = random_csr(rng, n, 40, hub_rows=[(3, 450), (499, 300)])
    val = rng.random(ci.size).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, val)
    plan = pkg.spmm.Plan(csr, 16, cost=cost, threads_per_wave=tpw, tiling=tiling, slab_bytes=slab_bytes, hot=hot)
    if tiling == "force":
        assert plan.info.num_slabs == -(-n // plan.info.slab_cols) and plan.info.slab_cols % 64 == 0
        # slabs narrower than the LDS table: every referenced column is hot, if asked for
        # (on its own the library does not spend a second launch on a matrix this small)
        assert plan.info.hot_rows == (1728 if hot == "force" else 0)
    else:
        assert plan.info.num_slabs == 1 and plan.info.hot_rows == 0
    check_plan_layout(pkg, orc, plan, rp, ci, val)
    # new values flow through set_values
    val2 = rng.random(ci.size).astype(np.float32)
    plan.set_values(torch.from_numpy(val2).to(dev))
    check_plan_layout(pkg, orc, plan, rp, ci, val2)
    plan.close()


@pytest.mark.parametrize("K,dtype,hot_rows", [(16, np.float32, 1728), (32, np.float16, 1472), (32, np.float32, 832),
                                              (64, np.float16, 704), (16, np.float16, 3456)])
def test_hot_columns_layout_and_result(pkg, orc, dev, K, dtype, hot_rows):
    """Slabs wider than the LDS table: part of every slab is hot, part cold."""
    g = pkg.graphs
    rp, ci, _ = g.generate("chunglu:n=9000,nnz=400000,gamma=2.1,dmax=3000", seed=21)
    n = rp.size - 1
    val = g.fill_uniform_f32(ci.size, 5, 0.0, 1.0).astype(dtype)
    X = g.fill_uniform_f32(n * K, 6, -1.0, 1.0).reshape(n, K).astype(dtype)
    csr = make_csr(pkg, dev, rp, ci, val)
    slab_cols = 4096
    # wider rows, fp16, or (here) a matrix whose hot gathers do not outweigh a second launch:
    # hot columns only on request
    auto = pkg.spmm.Plan(csr, K, cost=24, tiling="force", slab_bytes=slab_cols * K * val.itemsize)
    assert auto.info.hot_rows == 0
    auto.close()
    plan = pkg.spmm.Plan(csr, K, cost=24, tiling="force", slab_bytes=slab_cols * K * val.itemsize, hot="force")
    i = plan.info
    assert (i.num_slabs, i.slab_cols, i.hot_rows, i.num_segments) == (3, slab_cols, hot_rows, 6)
    assert 0 < i.hot_nnz < ci.size
    check_plan_layout(pkg, orc, plan, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    Y = plan.spmm(d_X)
    torch.cuda.synchronize()
    ref, scale = orc.spmm_f64(rp, ci, val.astype(np.float32), X.astype(np.float32), want_abs=True)
    if dtype == np.float32:
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    else:
        check_fp16(Y.cpu().numpy(), ref, scale)
    # the same plan without hot columns gives the same rows up to summation order
    cold = pkg.spmm.Plan(csr, K, cost=24, tiling="force", slab_bytes=slab_cols * K * val.itemsize, hot="off")
    assert cold.info.hot_rows == 0 and cold.info.num_segments == 3
    Yc = cold.spmm(d_X)
    torch.cuda.synchronize()
    if dtype == np.float32:
        check_fp32(Yc.cpu().numpy(), ref, scale, rel_elem=False)
    # twice in a row: bit-identical
    Y2 = plan.spmm(d_X)
    torch.cuda.synchronize()
    assert torch.equal(Y, Y2)


def test_plan_without_row_marks(pkg, orc, dev):
    """MPS_PLAN_NO_ROW_MARKS: plain column ids in the sliced array, and the kernel
    follows row_ptr as it does on the caller's CSR arrays (the path a matrix takes
    whose column ids and row-end counts do not fit 32 bits together)."""
    rng = np.random.default_rng(77)
    n, K = 700, 16
    rp, ci = random_csr(rng, n, 30, hub_rows=[(0, 650), (350, 400)])
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, K)) * 2 - 1).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    for tiling, slab_bytes in (("off", 0), ("force", 16384)):
        plan = pkg.spmm.Plan(csr, K, cost=12, tiling=tiling, slab_bytes=slab_bytes, hot="off", row_marks=False)
        assert plan.info.mark_shift == 0 and plan.info.hot_rows == 0
        check_plan_layout(pkg, orc, plan, rp, ci, val)
        Y = plan.spmm(d_X)
        torch.cuda.synchronize()
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
        plan.close()
    plan = pkg.spmm.Plan(csr, K, cost=12, tiling="off")
    assert plan.info.mark_shift == 10  # 700 columns: 10 bits
    plan.close()


@pytest.mark.parametrize("K,dtype", [(16, np.float32), (4, np.float32), (2, np.float32), (1, np.float32), (64, np.float16),
                                     (4, np.float16), (2, np.float16), (1, np.float16), (256, np.float32)])
def test_resident_columns_layout_and_result(pkg, orc, dev, K, dtype):
    """Untiled plan with resident columns (resident_bytes set, so that a small matrix gets them): the busiest
    columns' entries are plain, all others carry the streamed flag and are gathered with the streaming hint;
    the product has the same bits as without the flag (same partition, same order of summation).  The widths
    cover the 16-, 8-, 4- and 2-byte gathers of both element types."""
    rng = np.random.default_rng(1234 + K)
    n = 900
    rp, ci = random_csr(rng, n, 24, hub_rows=[(3, 800), (500, 650)])
    half = dtype == np.float16
    val = rng.random(ci.size).astype(dtype)
    X = (rng.random((n, K)) * 2 - 1).astype(dtype)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    row_bytes = K * (2 if half else 4)
    want = 40
    plan = pkg.spmm.Plan(csr, K, cost=12, tiling="off", resident_bytes=want * row_bytes)
    assert plan.info.resident_cols == want and plan.info.num_slabs == 1 and plan.info.mark_shift == 10
    check_plan_layout(pkg, orc, plan, rp, ci, val)
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    plain = pkg.spmm.Plan(csr, K, cost=12, tiling="off", resident="off")
    assert plain.info.resident_cols == 0
    Y0 = plain.spmm(d_X)
    torch.cuda.synchronize()
    assert torch.equal(Y, Y0)
    if half:
        ref, scale = orc.spmm_f64_f16in(rp, ci, val, X, want_abs=True)
        check_fp16(Y.cpu().numpy(), ref, scale)
    else:
        ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    # new values through the kept source indices
    val2 = rng.random(ci.size).astype(dtype)
    plan.set_values(to_dev(dev, val2)[0])
    plain.set_values(to_dev(dev, val2)[0])
    assert torch.equal(plan.spmm(d_X), plain.spmm(d_X))
    plan.close()
    plain.close()


@pytest.mark.parametrize("K,dtype,tiles", [(128, np.float32, True), (256, np.float32, True), (256, np.float16, True),
                                           (64, np.float32, False), (160, np.float32, True), (136, np.float32, False)])
def test_column_tiles_for_wide_rows(pkg, orc, dev, K, dtype, tiles):
    """Untiled plans for short matrix rows and rows of X of 512 bytes or more (a multiple of 128): lane-groups of 8
    lanes, one pass per 128 bytes of row pitch, the caller's merge items per wavefront kept (cost scaled by the
    groups per wavefront).  Same product as with full rows (other partition: equal within rounding) and as the
    oracle; explicit partitions per wavefront or MPS_PLAN_NO_COLUMN_TILES keep full rows."""
    rng = np.random.default_rng(4321 + K)
    n = 1200
    rp, ci = random_csr(rng, n, 28, hub_rows=[(7, 900)])
    half = dtype == np.float16
    val = rng.random(ci.size).astype(dtype)
    X = (rng.random((n, K)) * 2 - 1).astype(dtype)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    eb = 2 if half else 4
    full = pkg.spmm.Plan(csr, K, cost=96, column_tiles=False)
    plan = pkg.spmm.Plan(csr, K, cost=96)
    assert full.info.threads_per_wave == pkg.graphs.max_threads_per_wave(K, eb) and full.info.cost == 96
    if tiles:
        assert plan.info.threads_per_wave == 8 and plan.info.cost == max(16, 96 * full.info.threads_per_wave // 8)
    else:
        assert plan.info.threads_per_wave == full.info.threads_per_wave and plan.info.cost == 96
    assert pkg.spmm.Plan(csr, K, cost=96, threads_per_wave=1).info.threads_per_wave == 1
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    Y0 = full.spmm(d_X)
    torch.cuda.synchronize()
    if half:
        ref, scale = orc.spmm_f64_f16in(rp, ci, val, X, want_abs=True)
        check_fp16(Y.cpu().numpy(), ref, scale)
        check_fp16(Y0.cpu().numpy(), ref, scale)
    else:
        ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
        check_fp32(Y0.cpu().numpy(), ref, scale, rel_elem=False)
    assert torch.equal(Y, plan.spmm(d_X))
    check_plan_layout(pkg, orc, plan, rp, ci, val)


def test_resident_columns_are_chosen_for_large_skewed_inputs_only(pkg, dev):
    """Without resident_bytes the library flags streamed gathers only where they were measured to pay: X of
    192 MiB or more and at least 40 % of the nonzeros in the 10 MiB of busiest columns; a pitch that is not a
    power of two (64-bit offsets) never gets them."""
    rng = np.random.default_rng(5)
    rp, ci = random_csr(rng, 600, 20)
    val = rng.random(ci.size).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, val)
    assert pkg.spmm.Plan(csr, 16, tiling="off").info.resident_cols == 0           # small X
    assert pkg.spmm.Plan(csr, 20, tiling="off", resident_bytes=800).info.resident_cols == 0  # 80-byte pitch
    assert pkg.spmm.Plan(csr, 16, tiling="off", resident_bytes=64 * 10).info.resident_cols == 10


@pytest.mark.parametrize("mode", ["degree", "gcn"])
@pytest.mark.parametrize("K,tiling,slab_bytes,hot", [(16, "off", 0, "off"), (16, "force", 8192, "off"), (16, "force", 8192, "force"),
                                                     (20, "off", 0, "off"), (4, "force", 2048, "off"), (1, "off", 0, "off"),
                                                     (64, "off", 0, "off")])
def test_degree_weight_plans(pkg, orc, dev, mode, K, tiling, slab_bytes, hot):
    """Plans that form the reference's implicit edge weight deg(r) * deg(c) (src/MergePathSpMM.cu:450,459-460;
    or the GCN norm) from one factor per node instead of a value array: against the fp64 row loop over the
    oracle's weight array, for untiled, tiled and hot-column plans; with X = 1 (the reference's input,
    src/MergePathSpMM.cu:180-182) the product mode is exact integer arithmetic."""
    rng = np.random.default_rng(99 + K)
    n = 800
    rp, ci = random_csr(rng, n, 20, hub_rows=[(1, 700), (400, 300)])
    w = orc.degree_values(rp, ci, mode="product" if mode == "degree" else "gcn")
    X = (rng.random((n, K)) * 2 - 1).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, np.zeros(ci.size, dtype=np.float32))  # values must not be read
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, K, cost=12, tiling=tiling, slab_bytes=slab_bytes, hot=hot, weights=mode)
    assert (plan.info.num_slabs > 1) == (tiling == "force") and (plan.info.hot_rows > 0) == (hot == "force")
    assert plan.info.rowblock_steps == 0
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    torch.cuda.synchronize()
    ref, scale = orc.spmm_f64(rp, ci, w, X, want_abs=True)
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    assert torch.equal(Y, plan.spmm(d_X))
    if mode == "degree":
        deg = np.diff(rp).astype(np.int64)
        rows = np.repeat(np.arange(n), deg)
        want = deg * np.bincount(rows, weights=deg[ci], minlength=n).astype(np.int64)
        assert want.max() < 2 ** 24
        Y1 = plan.spmm(torch.ones_like(d_X)).cpu().numpy()
        assert np.array_equal(Y1, np.repeat(want[:, None], K, axis=1).astype(np.float32))
    with pytest.raises(pkg._cabi.MpsError) as e:
        plan.set_values(csr.val)
    assert e.value.status == pkg._cabi.MPS_ERR_UNSUPPORTED
    plan.close()


def test_degree_weight_plans_are_fp32_slab_plans(pkg, dev):
    rng = np.random.default_rng(8)
    rp, ci = random_csr(rng, 300, 12)
    half = make_csr(pkg, dev, rp, ci, np.zeros(ci.size, dtype=np.float16))
    with pytest.raises(pkg._cabi.MpsError) as e:
        pkg.spmm.Plan(half, 16, weights="degree")
    assert e.value.status == pkg._cabi.MPS_ERR_UNSUPPORTED
    full = make_csr(pkg, dev, rp, ci, np.zeros(ci.size, dtype=np.float32))
    with pytest.raises(pkg._cabi.MpsError) as e:
        pkg.spmm.Plan(full, 16, weights="degree", rowblock="force")
    assert e.value.status == pkg._cabi.MPS_ERR_UNSUPPORTED


def test_unsorted_rows(pkg, dev):
    n = 130  # two 64-column slabs
    rp = np.concatenate([[0, 3, 5], np.full(n - 2, 5)]).astype(np.int32)
    ci = np.array([100, 70, 0, 0, 129], dtype=np.int32)  # row 0 decreasing
    csr = make_csr(pkg, dev, rp, ci, np.ones(5, dtype=np.float32))
    with pytest.raises(pkg.MpsError) as e:
        pkg.spmm.Plan(csr, 16, cost=4, tiling="force", slab_bytes=4096)
    assert e.value.status == pkg._cabi.MPS_ERR_UNSORTED
    # a decrease exactly at a row boundary is fine, and so are repeated ids
    ci_ok = np.array([0, 70, 70, 0, 129], dtype=np.int32)
    csr = make_csr(pkg, dev, rp, ci_ok, np.ones(5, dtype=np.float32))
    assert pkg.spmm.Plan(csr, 16, cost=4, tiling="force", slab_bytes=4096).info.num_slabs == 3


def test_unsorted_rows_fall_back_to_untiled_in_auto_mode(pkg, orc, dev):
    g = pkg.graphs
    rp, ci, _ = g.generate("chunglu:n=120000,nnz=18000000,gamma=2.1,dmax=9000", seed=4)
    n, K = rp.size - 1, 16
    ci = ci.copy()
    lo, hi = rp[10], rp[11]
    ci[lo:hi] = ci[lo:hi][::-1]  # one row descending
    val = g.fill_uniform_f32(ci.size, 11, 0.0, 1.0)
    X = g.fill_uniform_f32(n * K, 13, -1.0, 1.0).reshape(n, K)
    csr = make_csr(pkg, dev, rp, ci, val)
    assert pkg.spmm.tile_shape(n, ci.size, K)[0] > 1
    plan = pkg.spmm.Plan(csr, K, cost=64)
    assert plan.info.num_slabs == 1
    (d_X,) = to_dev(dev, X)
    Y = plan.spmm(d_X)
    torch.cuda.synchronize()
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)


@pytest.mark.parametrize("K", [1, 4, 16, 20, 64, 256, 260])
def test_plan_spmm_against_oracle(pkg, orc, dev, K):
    rng = np.random.default_rng(100 + K)
    n = 900
    rp, ci = random_csr(rng, n, 60, hub_rows=[(0, 800), (450, 777), (899, 600)])
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, K)) * 2 - 1).astype(np.float32)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    for tiling, slab_bytes, cost, tpw in (("off", 0, 32, 0), ("force", 320 * K * 4, 32, 0), ("force", 128 * K * 4, 128, 0),
                                          ("force", 64 * K * 4, 7, 1), ("off", 0, 7, 0)):
        plan = pkg.spmm.Plan(csr, K, cost=cost, threads_per_wave=tpw, tiling=tiling, slab_bytes=slab_bytes)
        out = torch.full_like(d_X, float("nan"))
        Y = plan.spmm(d_X, out=out)
        torch.cuda.synchronize()
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
        again = plan.spmm(d_X, out=torch.empty_like(d_X))
        assert torch.equal(Y, again)  # deterministic
        plan.close()


def test_plan_edge_shapes(pkg, orc, dev):
    rng = np.random.default_rng(6)
    K = 16
    for deg in (np.array([300, 0, 0, 1, 2, 0]), np.array([0, 0, 5000, 0]), np.zeros(50, dtype=np.int64), np.array([9]),
                np.array([1, 1, 1, 1, 777]), np.array([0, 1, 0])):
        n = max(int(deg.size), int(deg.max()) if deg.size else 1, 16)
        deg_full = np.zeros(n, dtype=np.int64)
        deg_full[: deg.size] = deg
        rp = np.concatenate([[0], np.cumsum(deg_full)]).astype(np.int32)
        ci = np.concatenate([np.sort(rng.choice(n, size=int(d), replace=False)) for d in deg_full] +
                            [np.zeros(0, dtype=np.int64)]).astype(np.int32)
        val = rng.random(ci.size).astype(np.float32)
        X = (rng.random((n, K)) * 2 - 1).astype(np.float32)
        ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
        csr = make_csr(pkg, dev, rp, ci, val)
        (d_X,) = to_dev(dev, X)
        for tiling, sb, cost in (("off", 0, 1), ("off", 0, 64), ("force", 64 * K * 4, 5), ("force", 1024 * K * 4, 256)):
            plan = pkg.spmm.Plan(csr, K, cost=cost, tiling=tiling, slab_bytes=sb)
            Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan"))).cpu().numpy()
            check_fp32(Y, ref, scale, rel_elem=False)
            assert (Y[deg_full == 0] == 0).all()
            plan.close()


@pytest.mark.parametrize("num_slabs", [3, 5, 6, 7, 11])
def test_hot_launch_never_has_more_workgroups_than_cus(pkg, orc, dev, num_slabs):
    """One LDS table per CU: a hot launch of 258 workgroups on 256 CUs would run its last two alone."""
    g = pkg.graphs
    rp, ci, _ = g.generate("chunglu:n=60000,nnz=40000000,gamma=2.1,dmax=20000", seed=3)
    n, K = rp.size - 1, 16
    val = g.fill_uniform_f32(ci.size, 5, 0.0, 1.0)
    X = g.fill_uniform_f32(n * K, 6, -1.0, 1.0).reshape(n, K)
    csr = make_csr(pkg, dev, rp, ci, val)
    slab_cols = -(-(-(-n // num_slabs)) // 64) * 64
    plan = pkg.spmm.Plan(csr, K, tiling="force", slab_bytes=slab_cols * K * 4, hot="force")
    i = plan.info
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    assert i.num_slabs == num_slabs and i.hot_rows == 1728
    assert min(cus, i.hot_waves // 16) - num_slabs < i.hot_blocks <= cus  # all CUs busy, none twice
    (d_X,) = to_dev(dev, X)
    Y = plan.spmm(d_X)
    torch.cuda.synchronize()
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    plan.close()


def test_power_law_graph_auto_plan(pkg, orc, dev):
    g = pkg.graphs
    rp, ci, _ = g.generate("chunglu:n=100000,nnz=20000000,gamma=2.1,dmax=9000", seed=2)
    n, K = rp.size - 1, 16
    val = g.fill_uniform_f32(ci.size, 11, 0.0, 1.0)
    X = g.fill_uniform_f32(n * K, 13, -1.0, 1.0).reshape(n, K)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, K, cost=128, rowblock="off")
    assert plan.info.num_slabs == 2 and plan.info.slab_cols * K * 4 < (4 << 20)  # X = 6.4 MB: two slabs that fit an L2
    Y = plan.spmm(d_X)
    torch.cuda.synchronize()
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    # left to choose, the library builds a row-block plan: 26,000 nonzeros per block and step
    auto = pkg.spmm.Plan(csr, K)
    assert auto.info.rowblock_steps == 3 and auto.info.num_slabs == 1
    check_fp32(auto.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)
    auto.close()
    # the plain path on the caller's CSR agrees to rounding
    sched = pkg.spmm.generate_mp_sched(csr.row_ptr, csr.nnz, cost=128)
    Y0 = pkg.spmm.spmm_merge_path(csr, d_X, sched)
    assert (Y - Y0).abs().max().item() <= 1e-3


@pytest.mark.parametrize("spec,n_candidates,slab_sizes",
                         [("chunglu:n=20000,nnz=1500000,gamma=2.1,dmax=3000", 13, set()),
                          # X = 15.4 MB: slabs of 3 and 6 MiB are candidates too (X holds more than two of them)
                          ("chunglu:n=240000,nnz=12000000,gamma=2.1,dmax=5000", 15, {3 << 20, 6 << 20})])
def test_autotune_picks_a_measured_candidate(pkg, orc, dev, spec, n_candidates, slab_sizes):
    """mps_plan_autotune: every candidate is timed, the reported best is the
    fastest of them, and a plan built from it gives the right product."""
    g = pkg.graphs
    rp, ci, _ = g.generate(spec, seed=8)
    n, K = rp.size - 1, 16
    val = g.fill_uniform_f32(ci.size, 11, 0.0, 1.0)
    X = g.fill_uniform_f32(n * K, 13, -1.0, 1.0).reshape(n, K)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    best, tried = pkg.spmm.autotune(csr, d_X, repeats=3)
    assert len(tried) == n_candidates and all(t["ms"] > 0 for t in tried)
    assert {t["cost"] for t in tried} >= {16, 32, 64, 128, 256}
    assert {t["slab_bytes"] for t in tried if t["flags"] & pkg._cabi.MPS_PLAN_FORCE_TILING} == slab_sizes
    assert all(t["slab_bytes"] == 0 for t in tried if not t["flags"] & pkg._cabi.MPS_PLAN_FORCE_TILING)
    assert best["ms"] == min(t["ms"] for t in tried) and best in tried
    c = pkg._cabi
    tiling = "off" if best["flags"] & c.MPS_PLAN_NO_TILING else "force" if best["flags"] & c.MPS_PLAN_FORCE_TILING else "auto"
    hot = "off" if best["flags"] & c.MPS_PLAN_NO_HOT else "auto"
    # fp32, K = 16, X below 192 MiB: one candidate is a row-block plan, one a sweep plan, all others are slab plans
    assert sum(1 for t in tried if t["flags"] & c.MPS_PLAN_FORCE_ROWBLOCK) == 1
    assert sum(1 for t in tried if t["flags"] & c.MPS_PLAN_FORCE_SWEEP) == 1
    assert all(t["flags"] & (c.MPS_PLAN_FORCE_ROWBLOCK | c.MPS_PLAN_NO_ROWBLOCK | c.MPS_PLAN_FORCE_SWEEP) for t in tried)
    rowblock = "force" if best["flags"] & c.MPS_PLAN_FORCE_ROWBLOCK else "auto" if best["flags"] & c.MPS_PLAN_FORCE_SWEEP else "off"
    sweep = "force" if best["flags"] & c.MPS_PLAN_FORCE_SWEEP else "off"
    plan = pkg.spmm.Plan(csr, K, cost=best["cost"], threads_per_wave=best["threads_per_wave"], tiling=tiling, hot=hot,
                         slab_bytes=best["slab_bytes"], rowblock=rowblock, sweep=sweep)
    Y = plan.spmm(d_X)
    torch.cuda.synchronize()
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)


def test_plan_spmm_in_a_hip_graph(pkg, orc, dev):
    """mps_plan_spmm_* launches kernels only (no allocation, no memset, no
    synchronisation), so a caller can capture it: every replay, with other work
    and synchronisations between replays, gives the eager result bit for bit."""
    g = pkg.graphs
    K = 16
    for spec, kwargs in (("chunglu:n=20000,nnz=1500000,gamma=2.1,dmax=3000", dict(tiling="force", slab_bytes=4096 * K * 4)),
                         # with the hot launch (LDS tables) and its cold companion
                         ("chunglu:n=20000,nnz=1500000,gamma=2.1,dmax=3000",
                          dict(tiling="force", slab_bytes=4096 * K * 4, hot="force")),
                         # a row-block plan: gather kernel + main kernel
                         ("chunglu:n=20000,nnz=1500000,gamma=2.1,dmax=3000", dict(rowblock="force", rowblock_steps=5)),
                         # what the library picks by itself for this size: a row-block plan of one step
                         ("er:n=4096,deg=8", dict()), ("er:n=4096,deg=8", dict(rowblock="off"))):
        rp, ci, _ = g.generate(spec, seed=8)
        n = rp.size - 1
        val = g.fill_uniform_f32(ci.size, 11, 0.0, 1.0)
        csr = make_csr(pkg, dev, rp, ci, val)
        plan = pkg.spmm.Plan(csr, K, **kwargs)
        assert (plan.info.hot_rows > 0) == (kwargs.get("hot") == "force")
        assert (plan.info.rowblock_steps > 0) == (kwargs.get("rowblock") == "force" or not kwargs)
        X = torch.from_numpy(g.fill_uniform_f32(n * K, 13, -1.0, 1.0).reshape(n, K)).to(dev)
        Y = torch.full_like(X, float("nan"))
        eager = plan.spmm(X).clone()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            plan.spmm(X, out=Y)  # warm-up on the capture stream
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            plan.spmm(X, out=Y)
        for it in range(4):
            Y.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(Y, eager), "replay %d" % it
            X2 = X * (it + 2.0)  # eager work and a changed input between replays
            want2 = plan.spmm(X2).clone()
            torch.cuda.synchronize()
            X.copy_(X2)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(Y, want2), "replay with new input %d" % it
            eager = want2
        ref, scale = orc.spmm_f64(rp, ci, val, X.cpu().numpy(), want_abs=True)
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
        plan.close()


def test_plan_refuses_columns_beyond_the_matrix(pkg, dev):
    rng = np.random.default_rng(4)
    rp, ci = random_csr(rng, 500, 20)
    val = rng.random(ci.size).astype(np.float32)
    bad = ci.copy()
    bad[7] = 500  # one past the last row of X
    csr = make_csr(pkg, dev, rp, bad, val)
    for kwargs in (dict(), dict(tiling="force", slab_bytes=64 * 16 * 4), dict(tiling="force", slab_bytes=64 * 16 * 4, hot="force")):
        with pytest.raises(pkg._cabi.MpsError) as e:
            pkg.spmm.Plan(csr, 16, cost=8, **kwargs)
        assert e.value.status == pkg._cabi.MPS_ERR_INVALID_CSR
