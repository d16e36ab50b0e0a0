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


def test_program_against_the_cpp_surface_builds():
    """bam_amd/examples/array_sum.hip uses Controller / page_cache_t / range_t / array_t / array_d_t / bam_ptr the way
    the reference's benchmarks do; it has to compile for gfx950 and link against the library (no GPU needed for that)"""
    subprocess.run(["make", "-s", "-C", os.path.join(ROOT, "bam_amd", "csrc"), "../examples/array_sum"], check=True)
    exe = os.path.join(ROOT, "bam_amd", "examples", "array_sum")
    assert os.path.exists(exe) and os.access(exe, os.X_OK)
    syms = subprocess.run(["nm", "-D", "--undefined-only", exe], capture_output=True, text=True, check=True).stdout
    assert "bam_target_create" in syms and "nvm_ctrl_init" in syms or "nvmt_lookup" in syms or "bam_target_create" in syms
