"""bench.py's contract, as far as it can be checked without a GPU: one GPU only, the traffic figures of the
roofline come from the committed counter summary, and the profile summaries name commands that exist."""
import importlib.util
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)
    assert not r.stdout.strip().startswith("{")          # no result line for a run that measured nothing


def test_roofline_traffic_is_read_from_the_counter_summary():
    traffic = _bench().config4_traffic_bytes()
    assert set(traffic) >= {"buckets", "range"}
    algorithmic = 1_048_576 * (2 * 256 + 8)
    for layout, measured in traffic.items():
        # a Zipf batch re-reads hot rows from L2: below the algorithmic bytes, above the bytes written
        assert 268_435_456 < measured < algorithmic, layout
    assert traffic["buckets"] > traffic["range"]          # the bucket lines


def test_profile_summaries_name_commands_on_committed_files():
    flags = set(re.findall(r'"(--[a-z0-9-]+)"', open(os.path.join(ROOT, "bench.py")).read()))
    for name in sorted(os.listdir(os.path.join(ROOT, "profiles"))):
        text = open(os.path.join(ROOT, "profiles", name)).read()
        commands = [l.strip() for l in text.splitlines() if "rocprofv3" in l and " -- " in l]
        assert commands, name                             # every summary gives the command that made it
        for c in commands:
            program = c.split(" -- ", 1)[1]
            if program.startswith("$B"):                  # a shell variable defined on the line above the commands
                program = re.search(r'B="([^"]+)"', text).group(1)
            words = program.split()
            assert words[0] in ("python3", "python") and words[1] == "bench.py", (name, c)
            for w in words[2:]:
                if w.startswith("--"):
                    assert w in flags, (name, w)          # the flag exists in bench.py
            assert "_work" not in c and "--sys-trace" not in c and not ("--pmc" in c and "--kernel-trace" in c), (name, c)
