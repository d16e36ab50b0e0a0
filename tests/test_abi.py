"""The C-ABI libraries load and export every symbol the public headers declare (no compute calls: no GPU here)."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")


def _declared(header, prefix):
    text = open(os.path.join(INC, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    names = set(re.findall(r"\b(%s\w+)\s*\(" % prefix, text))
    # static inline helpers live in the header, not in the library
    inline = set(re.findall(r"static\s+inline\s+[\w\s\*]+?\b(%s\w+)\s*\(" % prefix, text))
    return names - inline


def test_host_library_exports_nvme_api():
    subprocess.run(["make", "-s", "-C", os.path.join(ROOT, "bam_amd", "csrc"), "host"], check=True)
    L = ctypes.CDLL(os.path.join(ROOT, "bam_amd", "libbam_host.so"))
    wanted = set()
    for h in ("nvm_ctrl.h", "nvm_dma.h", "nvm_aq.h", "nvm_admin.h", "nvm_queue.h", "nvm_error.h"):
        wanted |= _declared(h, "nvm_")
    wanted |= _declared("nvmt.h", "nvmt_")
    wanted -= {"nvm_ok"}
    assert len(wanted) > 30
    missing = [n for n in sorted(wanted) if not hasattr(L, n)]
    assert not missing, missing


def test_full_library_exports_every_declared_entry_point():
    from bam_amd import _lib
    path = _lib.lib_path()
    if not os.path.exists(path):
        pytest.skip("libbam_amd.so not built here (needs hipcc): build() compiles it")
    L = _lib.load()
    declared = _declared("bam_amd.h", "bam_")
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    for name in declared:
        assert hasattr(L, name), name
    # the host part is linked in as well
    for name in ("nvm_raw_ctrl_init", "nvm_aq_create", "nvmt_create", "nvm_admin_sq_create"):
        assert hasattr(L, name), name


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from bam_amd import _lib
    monkeypatch.setattr(_lib, "_LIB", None)
    monkeypatch.setattr(_lib, "_HERE", str(tmp_path))
    with pytest.raises(_lib.LibraryMissing):
        _lib.load()


def test_argument_checks_without_a_gpu():
    """Entry points validate their arguments before touching the device."""
    from bam_amd import _lib
    if not os.path.exists(_lib.lib_path()):
        pytest.skip("libbam_amd.so not built here")
    L = _lib.load()
    assert L.bam_array_read(None, 1, None, 1, 1, 64, None, None) != 0
    assert b"null" in L.bam_last_error()
    assert L.bam_gen_mod(1, 0, 10, 0, 1, None, None) != 0
    import errno
    # the entry points added for element-wise results, graph plans, launch shapes and measurements refuse null handles too
    assert L.bam_array_gather(None, 1, None, 1, 64, None, None) == errno.EINVAL and b"bam_array_gather" in L.bam_last_error()
    assert L.bam_array_set_graph(None, None, 0, None) == errno.EINVAL
    assert L.bam_bfs_shaped(None, None, 1, 0, None, 0, 1, 1, None, None) == errno.EINVAL
    assert L.bam_cc_shaped(None, None, 1, None, 0, 1, 1, None, None) == errno.EINVAL
    assert L.bam_atomic_pairs_kernel(None, None, 0, 1, None, None) == errno.EINVAL
    assert L.bam_xcd_relay(None, 0, 4096, 1, 1, 64, 0, None, None) == errno.EINVAL
    assert L.bam_scan_noalloc(None, 1, 64, None, None) == errno.EINVAL
    out = ctypes.c_void_p()
    assert L.bam_ctrl_create(ctypes.byref(out), b"/dev/not-published", 1, 0, 64, 1, 4096, 0) != 0
    assert b"no software NVMe target published" in L.bam_last_error() or b"HIP" in L.bam_last_error()
