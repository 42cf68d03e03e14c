"""bench.py takes the figures it cannot measure itself (profiler durations, HBM counters) from the rocprofv3 summaries
committed under profiles/.  These tests hold the parser and the summaries together: the rows bench.py looks for exist,
the numbers it derives are the ones the summaries' own text states, and the benchmark refuses a multi-GPU run."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def _text(path):
    with open(os.path.join(ROOT, path)) as f:
        return f.read()


def test_profiled_figures_come_from_the_committed_summaries():
    fig = bench.profiled_figures()
    assert 5.0 < fig["ffn_kernel_us"] < 20.0 and 2.0 < fig["gemv_4096_kernel_us"] < 8.0
    assert fig["fetch_scale"] == 2.0 and fig["write_scale"] == 1.0  # the factors the counter summary states
    # the traffic figure is the one the summary's own reading states (digits grouped with spaces there)
    grouped = f"{fig['ffn_traffic_bytes']:,}".replace(",", " ")
    assert grouped in _text(bench.PMC_MD), grouped
    # the kernel-trace row that the roofline cites is the one with the largest share of the run
    rows = [l for l in _text(bench.TRACE_MD).splitlines() if l.startswith("| ") and "%" not in l and "---" not in l]
    shares = {l.split("|")[1].strip(): float(l.split("|")[6]) for l in rows}
    assert max(shares, key=shares.get) == bench.FFN_KERNEL
    # algorithmic bytes of that launch as bench.py computes them: traffic within 3 % of it (no wasted re-reads)
    alg = 2 * bench.qweight_bytes(4096, 11008) + 2 * 4096 * 2 + 11008 * 2
    assert alg == 46888448
    assert 1.0 <= fig["ffn_traffic_bytes"] / alg <= 1.03


def test_every_profile_names_its_command_and_no_round():
    for name in os.listdir(os.path.join(ROOT, "profiles")):
        text = _text(os.path.join("profiles", name))
        assert "rocprofv3" in text and "bench.py" in text, name
        assert not re.search(r"\\bround\\s*\\d|_r\\d\\d", name), name


def test_bench_refuses_more_than_one_gpu():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0 and "ONE GPU" in res.stderr
