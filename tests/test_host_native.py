"""Builds and runs the native host-side checks (NVMe layer + software target); no GPU involved."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_native_host_checks(tmp_path):
    subprocess.run(["make", "-s", "-C", os.path.join(ROOT, "bam_amd", "csrc"), "host"], check=True)
    exe = tmp_path / "test_host"
    subprocess.run(["g++", "-std=c++17", "-O1", "-w", "-I", os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "native", "test_host.cpp"), "-o", str(exe),
                    "-L", os.path.join(ROOT, "bam_amd"), "-lbam_host", "-lpthread",
                    "-Wl,-rpath," + os.path.join(ROOT, "bam_amd")], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    oks = [l for l in r.stdout.splitlines() if l.startswith("ok ")]
    assert len(oks) >= 40 and "PASSED" in r.stdout
