"""Host-side checks of bench.py's command-line contract (no GPU): one GPU only, and the kernel-trace
summary that the profile summaries are made with."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          cwd=ROOT, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _bench("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)


def test_summarize_trace_reports_first_worst_and_settled_durations(tmp_path):
    # 100 dispatches of one kernel: 20 at 10 us, a dip of 40 at 15 us, 40 settled at 9 us; one other kernel
    rows = ["Kind,Kernel_Name,Start_Timestamp,End_Timestamp"]
    t = 1000
    for i in range(100):
        d = 10000 if i < 20 else (15000 if i < 60 else 9000)
        rows.append('KERNEL_DISPATCH,"void k<1, 2>(int)",%d,%d' % (t, t + d))
        t += d
    rows.append("KERNEL_DISPATCH,other,%d,%d" % (t, t + 500))
    path = tmp_path / "t_kernel_trace.csv"
    path.write_text("\n".join(rows) + "\n")
    r = _bench("--summarize-trace", str(path))
    assert r.returncode == 0, r.stderr
    lines = [json.loads(l) for l in r.stdout.splitlines() if l.startswith("{")]
    assert [l["kernel"] for l in lines] == ["void k<1, 2>(int)", "other"]  # by total time
    k = lines[0]
    assert k["dispatches"] == 100
    assert k["first20_median_us"] == 10.0 and k["worst40_median_us"] == 15.0 and k["last_quarter_median_us"] == 9.0
    assert abs(k["mean_us"] - (20 * 10 + 40 * 15 + 40 * 9) / 100) < 1e-9
