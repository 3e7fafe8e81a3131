"""CPU: the parts of bench.py's contract that need no GPU."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True, timeout=120)
    assert out.returncode == 2
    assert "ONE GPU" in out.stderr and out.stdout.strip() == ""


def test_flags_and_algorithmic_bytes():
    sys.path.insert(0, ROOT)
    import bench

    # nibbles + bf16 block scales + activations in + outputs out, per Linear
    assert bench.algorithmic_bytes(1, 1536, 8960, False) == 7_783_424
    assert bench.algorithmic_bytes(1, 1536, 151936, False) == 131_886_592
    total = 28 * sum(bench.algorithmic_bytes(1, K, N, b) for (_, K, N, b) in bench.LAYER_LINEARS)
    total += bench.algorithmic_bytes(1, *bench.LM_HEAD[1:])
    assert total == 873_717_248
    assert bench.PASS_TRAFFIC_BYTES_PER_LAUNCH >= total // 113      # traffic cannot be below the algorithmic bytes
    argv, sys.argv = sys.argv, ["bench.py"]
    try:
        args = bench.parse()
    finally:
        sys.argv = argv
    assert args.gpus == 1 and args.steps > 0 and args.warmup >= 0


def test_traffic_constant_is_the_one_the_counter_profile_derives():
    """roofline.traffic is typed into bench.py (a bench run cannot carry hardware counters): it must be the
    figure the committed counter summary arrives at, so that a kernel change that re-measures the one without
    updating the other is caught here."""
    sys.path.insert(0, ROOT)
    import bench
    import re

    text = open(os.path.join(ROOT, "profiles", "traffic_fetch_write_decode_prefill.md")).read()
    m = re.search(r"Traffic per launch = ([\d,]+) \+ ([\d,]+) = ([\d,]+) bytes", text)
    assert m, "the profile no longer states the traffic per launch"
    fetch, write, total = (int(x.replace(",", "")) for x in m.groups())
    assert fetch + write == total == bench.PASS_TRAFFIC_BYTES_PER_LAUNCH
    # and the profiled command times the pass the bench line's value comes from
    assert "--roofline-only --pass split" in text
