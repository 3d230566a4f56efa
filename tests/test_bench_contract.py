"""CPU-only checks of bench.py's contract: the argument parser, the refusal of more than one GPU, and that every HBM
traffic figure it carries (PMC_TRAFFIC_BYTES, typed in from rocprofv3 counter runs) is backed by the counter values
written down in profiles/: a figure that no summary holds has gone stale."""
import ast
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _traffic_terms():
    """{key: [KiB literals]} from the PMC_TRAFFIC_BYTES expression in bench.py, without importing it."""
    tree = ast.parse(open(os.path.join(ROOT, "bench.py")).read())
    for node in tree.body:
        if isinstance(node, ast.Assign) and getattr(node.targets[0], "id", "") == "PMC_TRAFFIC_BYTES":
            out = {}
            for k, v in zip(node.value.keys, node.value.values):
                lits = [n.value for n in ast.walk(v) if isinstance(n, ast.Constant) and isinstance(n.value, float)]
                out[k.value] = [x for x in lits if x not in (1.0, 2.0)]
            return out
    raise AssertionError("bench.py has no PMC_TRAFFIC_BYTES")


def test_traffic_figures_are_backed_by_the_profile_summaries():
    text = ""
    for f in sorted(os.listdir(os.path.join(ROOT, "profiles"))):
        text += open(os.path.join(ROOT, "profiles", f)).read()
    numbers = set(float(m.replace(",", "").rstrip(".")) for m in re.findall(r"\d[\d,]*(?:\.\d+)?", text))
    terms = _traffic_terms()
    assert len(terms) >= 8
    for key, kib in terms.items():
        assert kib, key
        for v in kib:
            assert v in numbers, f"{key}: {v} KiB is in bench.py but in no file under profiles/"


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr) or "1 GPU" in (r.stdout + r.stderr) or "single" in (r.stdout + r.stderr).lower()
