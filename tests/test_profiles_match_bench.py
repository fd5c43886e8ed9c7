"""The figures bench.py quotes from the committed rocprofv3 summaries must be the ones the summaries hold: a
profile that is refreshed without the table in bench.py (or the other way round) fails here."""
import importlib.util
import re
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def _bench():
    spec = importlib.util.spec_from_file_location("helix_bench", ROOT / "bench.py")
    mod = importlib.util.module_from_spec(spec)
    sys.modules["helix_bench"] = mod
    spec.loader.exec_module(mod)
    return mod


def test_traffic_table_equals_the_profile_summaries():
    bench = _bench()
    assert bench.MEASURED_TRAFFIC_BYTES, "no traffic rows"
    for (kernel, workload, channels), traffic in bench.MEASURED_TRAFFIC_BYTES.items():
        text = (ROOT / "profiles" / f"{kernel}_{workload}.md").read_text()
        assert f"{channels} channels" in text.splitlines()[0], f"{kernel} {workload}: channel count of the summary"
        # the first "total ... bytes" line is the leg with one set of tensors (the one `roofline.traffic` quotes)
        m = re.search(r"^\* total ([\d,]+) bytes = ([\d.]+) x the ([\d,]+) algorithmic bytes", text, re.M)
        assert m, f"{kernel} {workload}: no traffic total in the summary"
        assert int(m.group(1).replace(",", "")) == traffic, f"{kernel} {workload}: bench.py quotes {traffic}, the summary {m.group(1)}"
        # and the summary's algorithmic bytes are what bench.py computes for that workload
        sys.path.insert(0, str(ROOT))
        from helix_workloads import WORKLOADS
        w = WORKLOADS[workload]
        algo = w.combine_bytes(channels) if "combine" in kernel else w.exchange_bytes(channels)
        assert int(m.group(3).replace(",", "")) == algo
        assert abs(traffic / algo - float(m.group(2))) < 1e-3


def test_every_kernel_summary_names_a_command_of_committed_files():
    for path in sorted((ROOT / "profiles").glob("helix_*_kernel_*.md")):
        text = path.read_text()
        cmds = re.findall(r"-- (python3 \S+)", text)
        assert cmds, f"{path.name}: no command"
        for c in cmds:
            assert (ROOT / c.split()[1]).exists(), f"{path.name}: {c} is not a committed file"
        assert "_work" not in text
