"""bench.py without a GPU: the lookup of measured HBM traffic by plan signature, and the refusal of more than one GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def test_traffic_is_looked_up_by_plan_signature_and_names_its_profile():
    table = open(bench.TRAFFIC_TABLE).read()
    rows = [l for l in table.splitlines() if l.startswith("| `")]
    assert len(rows) >= 10
    for line in rows:
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        sig = cells[0].replace("`", "").replace(";", "|")
        traffic, where = bench.measured_traffic(sig)
        want = int((float(cells[2]) * float(cells[3]) + float(cells[4]) * float(cells[5])) * 1024)
        assert traffic == want and traffic > 0
        assert where.startswith("profiles/") and os.path.exists(os.path.join(ROOT, where))
    # the headline workload with the library's own plan has a row; a plan of another shape has none
    assert any(l.startswith("| `%s;rowblock;" % bench.HEADLINE) for l in rows)
    assert bench.measured_traffic(bench.HEADLINE + "|rowblock|steps=99|table_rows=1|blocks=1|cold_index_bits=0") == (None, None)


def test_hit_rate_comes_from_the_same_row_and_old_rows_have_none():
    table = open(bench.TRAFFIC_TABLE).read()
    seen_rate = False
    for line in table.splitlines():
        if not line.startswith("| `"):
            continue
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        sig = cells[0].replace("`", "").replace(";", "|")
        traffic, rate, where = bench.measured_counters(sig)
        assert traffic and where
        if len(cells) == 9:
            assert rate == round(float(cells[6]) / (float(cells[6]) + float(cells[7])), 4) and 0.0 < rate < 1.0
            seen_rate = True
        else:
            assert len(cells) == 7 and rate is None
    assert seen_rate
    assert bench.measured_counters("no such plan") == (None, None, None)
    assert bench.measured_counters("no such plan", with_requests=True, other_lines=5) == (None, None, None, None)


def test_gather_hit_rate_leaves_out_the_lines_that_are_read_once():
    info = FakeInfo(sweep_panels=256, sweep_slots=16932864, sweep_tiles=1, device_bytes=0)

    class W:
        n, K, eb = 1 << 20, 16, 4

    once = bench.lines_read_once(W, info)
    assert once == (8 * 16932864 + (1 << 20) * 64) // 128
    # the row of the table that holds this workload's sweep plan, whatever its panels look like today
    rows = [line.split("|")[1].strip().strip("`") for line in open(bench.TRAFFIC_TABLE) if line.startswith("| `rmat_s20_f32_k16;sweep;")]
    assert len(rows) == 1
    sig = rows[0].replace(";", "|")
    traffic, rate, where, gathers = bench.measured_counters(sig, with_requests=True, other_lines=once)
    assert traffic and where and rate < gathers < 1.0
    # slab plans write partial rows and read them again: no such estimate
    assert bench.lines_read_once(W, FakeInfo()) is None and bench.lines_read_once(W, None) is None


class FakeInfo:
    def __init__(self, **kw):
        self.sweep_panels = self.sweep_split_rows = self.rowblock_steps = self.rowblock_blocks = 0
        self.rowblock_local_tables = self.hot_rows = 0
        self.num_slabs = 1
        self.__dict__.update(kw)


def test_phases_that_launch_nothing_have_no_kernel():
    k = bench.kernels_of(FakeInfo(sweep_panels=256), 256)
    assert k == {"PREPARE": None, "MAIN": "sw_spmm_kernel", "FIXUP": None, "REDUCE": None}
    assert bench.kernels_of(FakeInfo(sweep_panels=512, sweep_split_rows=1), 256)["FIXUP"] == "sw_fixup_kernel"
    k = bench.kernels_of(FakeInfo(rowblock_steps=16, rowblock_blocks=256), 256)
    assert k == {"PREPARE": "rb_gather_hot_kernel", "MAIN": "rb_spmm_kernel", "FIXUP": None, "REDUCE": None}
    # one step, one round of blocks, or tables of a block's own: the table comes from X inside the main kernel
    assert bench.kernels_of(FakeInfo(rowblock_steps=1, rowblock_blocks=256), 256)["PREPARE"] is None
    assert bench.kernels_of(FakeInfo(rowblock_steps=1, rowblock_blocks=512, rowblock_local_tables=1), 256)["PREPARE"] is None
    assert bench.kernels_of(FakeInfo(rowblock_steps=1, rowblock_blocks=512), 256)["PREPARE"] == "rb_gather_hot_kernel"
    k = bench.kernels_of(FakeInfo(num_slabs=5, hot_rows=1728), 256)
    assert k["REDUCE"] == "tile_reduce_kernel" and k["FIXUP"] == "mp_fixup_kernel" and "hot + cold" in k["MAIN"]
    assert bench.kernels_of(FakeInfo(), 256)["REDUCE"] is None
    assert bench.kernels_of(None, 256)["MAIN"] == "mp_spmm_kernel"


def test_workloads_cover_the_benchmark_configurations():
    assert bench.HEADLINE in bench.WORKLOADS and len(bench.OTHER_CONFIGS) == 8
    assert all(w in bench.WORKLOADS for w in bench.OTHER_CONFIGS)
    ks = sorted(bench.WORKLOADS[w][1] for w in bench.OTHER_CONFIGS if w.startswith("rmat_s20"))
    assert ks == [16, 32, 64, 128, 256]
    # algorithmic bytes: row_ptr + col_idx + val + X + Y
    assert bench.algorithmic_bytes(232965, 114604189, 16, 4, 4) == 947584896


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert p.returncode != 0 and "one GPU" in p.stderr
