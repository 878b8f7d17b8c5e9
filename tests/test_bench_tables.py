"""bench.TRAFFIC_BYTES (the HBM bytes per launch that the benchmark reports as roofline.traffic)
is a copy of the counter summaries under profiles/: this test reads the summaries' tables and
fails when the two differ, so the constants cannot outlive a kernel change unnoticed."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def traffic_rows(name):
    """(kernel, grid threads, total bytes) of every table row of a profiles/*_hbm_traffic.md file"""
    rows = []
    for line in open(os.path.join(ROOT, "profiles", name)):
        m = re.match(r"\|\s*`([^`]+)`\s*\|\s*(\d+)\s*\|(.*)\|\s*(\d+)\s*\|\s*$", line)
        if m:
            rows.append((m.group(1), int(m.group(2)), int(m.group(4))))
    return rows


def test_traffic_constants_equal_the_profile_summaries():
    import bench
    decode = traffic_rows("decode_s2_planned_fused_hbm_traffic.md")
    prefill = traffic_rows("prefill_c3_hbm_traffic.md")
    assert decode and prefill
    seen = 0
    for key, total in bench.TRAFFIC_BYTES.items():
        kernel = key[-1]
        table = decode if key[0] == "s2" else prefill
        cands = [r for r in table if r[0] == kernel]
        assert cands, f"{kernel} is not in the profile summary"
        # a kernel that the step launches in two sizes (q/k/v and o): the constant is the larger launch
        row = max(cands, key=lambda r: r[1])
        assert row[2] == total, (key, row, total)
        seen += 1
    assert seen == len(bench.TRAFFIC_BYTES) >= 6
