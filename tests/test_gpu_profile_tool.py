"""The profile tool (the role of reference cpp_examples/profile.cc:17-36) on the device: it loads
a checkpoint object or a single graph file through the C++ host API, fingerprints and profiles
every operator, and prints the profiled running times."""
import json
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOOL = os.path.join(ROOT, "attention_superoptimizer_amd", "mirage_profile")
CHECKPOINT = os.path.join(ROOT, "tests", "golden", "gqa_spec_decode_checkpoint_excerpt.json")


def _run(*args):
    assert os.path.exists(TOOL), "mirage_profile is built by attention_superoptimizer_amd.build"
    p = subprocess.run([TOOL, *args], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stderr[-2000:]
    return p.stdout


def test_checkpoint_graphs_are_profiled():
    n = len(json.load(open(CHECKPOINT))["generated_graphs"])
    out = _run(CHECKPOINT)
    times = [float(t) for t in re.findall(r"graph \d+: \d+ operators, profiled running time: ([0-9.e+-]+) ms", out)]
    assert len(times) == n and all(0.0 < t < 1.0 for t in times), out[-1000:]
    m = re.search(r"(\d+) graphs: min ([0-9.e+-]+) ms, median ([0-9.e+-]+) ms, max ([0-9.e+-]+) ms", out)
    assert m and int(m.group(1)) == n
    assert float(m.group(2)) == pytest.approx(min(times), rel=1e-3)
    assert float(m.group(4)) == pytest.approx(max(times), rel=1e-3)
    print(out.splitlines()[-1], flush=True)


def test_a_range_and_a_single_graph_file(tmp_path):
    out = _run(CHECKPOINT, "2", "3")
    assert re.findall(r"graph (\d+):", out) == ["2", "3", "4"]
    # one graph written as a file of its own: printed back as JSON, then its time
    graph = json.load(open(CHECKPOINT))["generated_graphs"][0]
    path = tmp_path / "graph.json"
    path.write_text(json.dumps(graph))
    out = _run(str(path))
    assert "Profiled running time:" in out
    printed = json.loads(out[:out.index("Profiled running time:")])
    assert len(printed) == len(graph)
    assert [op["op_type"] for op in printed] == [op["op_type"] for op in graph]
