"""The barrier protocol among the workgroups of one XCD (lightseq_amd/csrc/xcd_sync.h) run as a
host model, one thread per workgroup: rounds complete with consistent data, a second launch
continues from the counters of the first, counters may wrap, and -- the case no GPU test may
provoke -- a workgroup that never arrives makes every waiter give up after a bounded number of
polls instead of spinning."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_xcd_barrier_protocol_host_model(tmp_path):
    exe = os.path.join(str(tmp_path), "xcd_sync_model")
    src = os.path.join(ROOT, "tests", "xcd_sync_model.cpp")
    subprocess.run(["g++", "-O2", "-std=c++17", "-pthread", "-o", exe, src], check=True)
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(p.stdout)
    assert p.returncode == 0, p.stdout
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 4 and all(": ok" in l for l in lines), p.stdout
