"""bench.py takes roofline.traffic from the committed rocprofv3 summary (profiles/bench_hbm_traffic_pmc.txt) instead of
constants in its source: the lines it parses must agree with the table of the same file, name the kernels by the labels the
library reports, and cover every configuration's dominant kernel."""
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_traffic_lines_parse_and_match_the_table_of_the_same_file():
    import bench
    traffic = bench.load_traffic()
    assert set(traffic) == {"c1", "c2_permute", "c2_reduce", "c3", "c4"}
    text = open(bench.TRAFFIC_FILE).read()
    rows = {}
    for line in text.splitlines():
        m = re.match(r"^(\S.*?)\s+(\d+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s*$", line)
        if m:
            rows[m.group(1)] = (float(m.group(5)), float(m.group(6)))   # read MB, written MB
    assert len(rows) >= 8
    for key, (nbytes, label) in traffic.items():
        assert label.startswith("(") and label.endswith(")") and "::" not in label
        name = label[1:-1]
        # the table cuts long names at 100 characters
        match = [v for k, v in rows.items() if k.startswith(name[:90])]
        assert len(match) == 1, (key, label, list(rows))
        assert abs((match[0][0] + match[0][1]) * 1e6 - nbytes) <= 0.06e6 * 2, (key, match[0], nbytes)
    # algorithmic bytes of the bandwidth-bound kernels: traffic within 1 % of them
    assert abs(traffic["c2_permute"][0] / (2 * 16 ** 6 * 8) - 1) < 0.01
    assert abs(traffic["c2_reduce"][0] / (16 ** 6 * 8 + 16 ** 4 * 8) - 1) < 0.01
    # a label that does not match the kernel that ran gives no figure
    assert bench.traffic_of("c3", "(some_other_kernel<double>)") is None
    assert bench.traffic_of("c3", traffic["c3"][1]) == traffic["c3"][0]


def test_profile_summaries_name_their_commands_and_no_working_files():
    pdir = os.path.join(ROOT, "profiles")
    files = sorted(f for f in os.listdir(pdir) if f.endswith((".txt", ".md")))
    assert files, "no profile summaries committed"
    for f in files:
        text = open(os.path.join(pdir, f)).read()
        # every summary states the command that made it, and that command runs committed files only
        if f.startswith("host_overhead"):
            assert "python3 bench.py --host-overhead" in text, f
        elif f.startswith("shape_sweep"):
            assert "python3 bench.py --shape-sweep" in text, f
        else:
            assert "rocprofv3 " in text and " -- python3 bench.py" in text, f
        assert "_work/" not in text, f
        assert os.path.getsize(os.path.join(pdir, f)) < 32 * 1024, f
