"""The drop-in claim, by compilation: the text of the reference's benchmark kernels, read from the reference tree at test
time (never committed; written to a temporary directory), is compiled for gfx950 in a translation unit that includes only
this repository's include/ headers.  Skipped where the reference tree is absent (the GPU box).  No GPU is needed.

What a maintainer of the reference has to touch is listed in EDITS and nowhere else: a kernel that does not appear there
compiles letter for letter."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"

# (namespace, file under the reference tree, [(first line, last line), ...]) - the kernels of the five benchmarks:
# array: sequential_access_kernel / random_access_kernel; block: sequential_access_kernel; cache: random_access_warp /
# sequential_access_warp; bfs: kernel_coalesce_coarse_ptr_pc; cc: cc_compute + kernel_coalesce_coarse_ptr_pc
KERNELS = [
    ("ref_array", "benchmarks/array/main.cu", [(43, 65)]),
    ("ref_block", "benchmarks/block/main.cu", [(99, 148)]),
    ("ref_cache", "benchmarks/cache/main.cu", [(44, 114)]),
    ("ref_bfs", "benchmarks/bfs/main.cu", [(655, 689)]),
    ("ref_cc", "benchmarks/cc/main.cu", [(123, 144), (595, 617)]),
]

# textual edits, applied to the extracted lines: (namespace, pattern, replacement, why)
EDITS = [
    ("ref_block", r"__shfl_sync\(0xFFFFFFFF,", "__shfl_sync(0xFFFFFFFFFFFFFFFFull,",
     "HIP's __shfl_sync takes a 64-bit lane mask (a wave has 64 lanes) and refuses a 32-bit one at compile time"),
    ("*", r"__launch_bounds__\((\d+),\s*\d+\)", r"__launch_bounds__(\1)",
     "the second argument is CUDA's minimum of resident blocks per SM; hipcc reads it as waves per SIMD, of which a "
     "gfx950 SIMD holds eight"),
]

# what the benchmarks' own main.cu files define around the kernels (settings.h enums, graph typedefs, the warp geometry):
# the only values that change are the two that say how wide a wave is
PRELUDE = r"""
#define HIP_ENABLE_WARP_SYNC_BUILTINS 1
#include <hip/hip_runtime.h>
#include <nvm_ctrl.h>
#include <nvm_types.h>
#include <nvm_queue.h>
#include <nvm_util.h>
#include <nvm_admin.h>
#include <nvm_error.h>
#include <nvm_cmd.h>
#include <ctrl.h>
#include <buffer.h>
#include <event.h>
#include <queue.h>
#include <nvm_parallel_queue.h>
#include <page_cache.h>
#include <util.h>
enum { READ = 0, WRITE = 1, MIXED = 2 };     /* benchmarks/block/settings.h */
enum { ORIG = 0, BAM_PTR_KIND = 1 };         /* benchmarks/cache/settings.h: ORIG selects operator[], anything else bam_ptr */
typedef uint64_t EdgeT;                      /* benchmarks/bfs/main.cu, benchmarks/cc/main.cu */
#define WARP_SHIFT 6                         /* 5 in the reference: a warp of 32 */
#define WARP_SIZE 64                         /* 32 in the reference */
#define BLOCK_NUM 1024ULL
#define MYINFINITY 0xFFFFFFFF
"""

# every template is instantiated and every kernel's address taken, so that nothing is left unchecked for want of a use
USES = r"""
void* bam_reference_kernels[] = {
    (void*)ref_array::sequential_access_kernel, (void*)ref_array::random_access_kernel,
    (void*)ref_block::sequential_access_kernel,
    (void*)ref_cache::random_access_warp<uint64_t>, (void*)ref_cache::sequential_access_warp<uint64_t>,
    (void*)ref_bfs::kernel_coalesce_coarse_ptr_pc, (void*)ref_cc::kernel_coalesce_coarse_ptr_pc,
};
"""


def _extract(path, ranges):
    with open(path, errors="replace") as f:
        lines = f.readlines()
    return "".join("".join(lines[a - 1:b]) + "\n" for a, b in ranges)


@pytest.mark.skipif(not os.path.isdir(REF), reason="the reference tree is not here")
def test_reference_benchmark_kernels_compile_against_include(tmp_path):
    parts = [PRELUDE]
    touched = set()
    for ns, rel, ranges in KERNELS:
        text = _extract(os.path.join(REF, rel), ranges)
        for who, pat, rep, _why in EDITS:
            if who in ("*", ns):
                text, n = re.subn(pat, rep, text)
                if n:
                    touched.add((ns, pat))
        parts.append("namespace %s {\n%s\n}\n" % (ns, text))
    parts.append(USES)
    tu = tmp_path / "reference_kernels.hip"
    tu.write_text("".join(parts))
    r = subprocess.run(["/opt/rocm/bin/hipcc", "-std=c++17", "-O3", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                        "-Wno-unused-value", "-I", os.path.join(ROOT, "include"), "-c", str(tu), "-o", str(tmp_path / "reference_kernels.o")],
                       capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-4000:]
    # the list of edits is the whole of it: the 64-bit mask in one kernel, the launch bounds where a kernel has two
    assert ("ref_block", EDITS[0][1]) in touched
    syms = subprocess.run(["nm", str(tmp_path / "reference_kernels.o")], capture_output=True, text=True).stdout
    for name in ("sequential_access_kernel", "random_access_kernel", "random_access_warp", "sequential_access_warp", "kernel_coalesce_coarse_ptr_pc"):
        assert name in syms, name
