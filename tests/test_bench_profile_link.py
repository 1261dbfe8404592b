"""bench.py's link to the tracked counter summary: the HBM-bytes table, the commit and the kernel-source hash it was taken on
are read back from profiles/ as written (no GPU needed)."""
import re

import bench
from crusaderbackend_amd import bench_report


def test_traffic_table_commit_and_source_hash_are_read_from_the_profile():
    table, commit, src_hash = bench.measured_hbm_bytes()
    assert table, "profiles/ holds the per-call HBM bytes of the benchmark step"
    assert all(v > 0 for v in table.values())
    assert commit and re.fullmatch(r"[0-9a-f]{7,40}", commit)
    # the hash is the line's value, not the name of the function that computes it
    assert src_hash and re.fullmatch(r"[0-9a-f]{16}", src_hash)
    assert re.fullmatch(r"[0-9a-f]{16}", bench_report.csrc_hash())
