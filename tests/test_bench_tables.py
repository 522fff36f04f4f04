"""bench.py's tracked inputs are current: every row of profiles/hbm_traffic.md was measured on the kernel source that
is in the tree (a stale row would silently turn `roofline.traffic` into null in the bench line). CPU only."""
import re
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))


def test_traffic_table_rows_match_the_kernel_sources_in_the_tree():
    import profile_tables as bench
    text = bench.TRAFFIC_FILE.read_text()
    rows = re.findall(r"^\|\s*(\w+)\s*\|\s*(\d+)\s*\|\s*\d+\s*\|\s*\d+\s*\|\s*([0-9a-f]{16})\s*\|", text, re.M)
    assert {(w, int(n)) for w, n, _ in rows} >= {("sgemm", 8192), ("scan", 1 << 30), ("gemm_bf16", 8192), ("add_m", 1 << 28)}
    for workload, size, digest in rows:
        assert digest == bench.source_hash(workload), (
            f"profiles/hbm_traffic.md: the {workload} row was measured on another version of "
            f"{bench.KERNEL_SOURCE[workload]}; re-run the two counter passes and `python bench.py --traffic-summary`")
        assert bench.measured_traffic(workload, int(size)) is not None
