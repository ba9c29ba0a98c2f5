"""bench.py's `roofline.traffic` figures are measured offline and kept in profiles/; a figure is
reported only while the kernel source it was measured on is unchanged."""

import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("k3q_bench", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_committed_traffic_figures_follow_the_recorded_sources():
    # every figure of the committed file is reported exactly when the sources recorded with it are
    # the sources in the tree (a kernel edited after its profile shows up as null, not as a failure)
    bench = _bench()
    with open(bench.TRAFFIC_FILE) as f:
        table = json.load(f)
    now = bench.sources_digest()
    changed = {n for n in now if table["_sources"].get(n) != now[n]}
    for key in table:
        if key.startswith("_"):
            continue
        files = next(v for k, v in bench.TRAFFIC_SOURCES.items() if key.startswith(k))
        fresh = not (set(files) | {"k3q_common.h"}) & changed
        assert bench.measured_traffic(key) == (table[key] if fresh else None), key


def test_a_changed_kernel_source_withholds_its_figures(tmp_path):
    bench = _bench()
    with open(bench.TRAFFIC_FILE) as f:
        table = json.load(f)
    table["_sources"]["k3q_gemm_i8.hip"] = "0" * 64
    stale = tmp_path / "traffic.json"
    stale.write_text(json.dumps(table))
    bench.TRAFFIC_FILE = str(stale)
    assert bench.measured_traffic("gemm_mfma_i8_M4096_K8192_N8192") is None
    assert bench.TRAFFIC_STALE == {"k3q_gemm_i8.hip"}
    assert bench.measured_traffic("gemv_w4s_M1_per_channel") == table["gemv_w4s_M1_per_channel"]
    assert bench.measured_traffic("no_such_kernel") is None
