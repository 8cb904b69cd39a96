"""The benchmark script's own bookkeeping, without a GPU: the one-GPU rule, the algorithmic byte counts it divides by,
and what it quotes from the committed counter summaries."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert run.returncode != 0
    assert "one GPU" in run.stderr and "--gpus must be 1" in run.stderr


def test_algorithmic_bytes_are_the_contract_figures():
    """The per-environment figures the scope contract states for the published configurations (4-byte words; links,
    coordinates, contact points, floating root)."""
    assert bench.algorithmic_bytes(8, 7, 0, False) == (396, 900)   # the contract's own sum for the chain (392, 896) leaves out the contact count word
    assert bench.algorithmic_bytes(13, 18, 4, True) == (864, 5472)
    assert bench.algorithmic_bytes(31, 36, 12, True) == (1960, 23272)
    assert bench.algorithmic_bytes(65, 64, 64, False) == (4640, 136736)
    assert bench.solver_bytes(36, 12) == 10944


def test_counter_summaries_are_quoted_with_their_source_and_their_age():
    digest = bench.solver_source_digest()
    assert len(digest) == 16 and int(digest, 16) >= 0
    for name, envs in (("humanoid", 4096), ("quadruped", 4096), ("humanoid", 65536), ("rope64", 8192)):
        figures = bench.profiled_figures(name, envs)
        assert figures is not None, f"profiles/counters_{name}_{envs}.txt holds no figures line"
        assert figures["from"] == os.path.join("profiles", f"counters_{name}_{envs}.txt")
        assert figures["taken_on_this_source"] == (figures["solver_source_sha256"] == digest)
        assert figures["traffic_bytes_per_launch"] > 0 and figures["valu_instructions_per_env"] > 0
        with open(os.path.join(ROOT, figures["from"])) as summary:
            text = summary.read()
        assert "rocprofv3 --pmc FETCH_SIZE" in text and "bench.py --only" in text   # every summary carries its commands
    assert bench.profiled_figures("no_such_workload", 1) is None
    json.dumps(bench.profiled_figures("humanoid", 4096))
