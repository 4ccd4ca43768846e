"""The HIP plugin against the reference's OWN headers.

Two checks, both on the CPU, both skipped where the reference tree is absent:
  * nixl_amd/csrc/plugin/hip_backend.cpp compiles (-fsyntax-only) with the reference's
    src/api/cpp, src/api/cpp/backend, src/core/telemetry and src/utils on the include path;
    the one header not taken from the reference is common/nixl_log.h (abseil logging there,
    iostream here).
  * tests/cpp/abi_layout_probe.cpp prints sizes, member offsets and virtual-table slots of
    every type that crosses the plugin boundary; built against the reference's headers and
    against include/nixl it must print the same text.
Reference: src/api/cpp/backend/backend_engine.h:33-251, backend_plugin.h:36-57,
backend_aux.h:30-208, nixl_descriptors.h.
"""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"
REF_INCLUDES = [os.path.join(REF, p) for p in ("src/api/cpp", "src/api/cpp/backend", "src/core/telemetry", "src/utils")]

pytestmark = pytest.mark.skipif(not all(os.path.isdir(p) for p in REF_INCLUDES),
                                reason="the reference tree is not present on this machine")


@pytest.fixture()
def shim_dir(tmp_path):
    """A directory that holds nothing but common/nixl_log.h, placed first on the include path."""
    os.makedirs(tmp_path / "shim" / "common")
    shutil.copy(os.path.join(ROOT, "include", "nixl", "common", "nixl_log.h"), tmp_path / "shim" / "common" / "nixl_log.h")
    return str(tmp_path / "shim")


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, " ".join(cmd) + "\n" + proc.stdout
    return proc.stdout


def test_plugin_source_compiles_against_reference_headers(shim_dir):
    rocm_include = "/opt/rocm/include"
    if not os.path.isdir(rocm_include):
        pytest.skip("no ROCm headers")
    cmd = ["g++", "-std=c++20", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", "-I" + shim_dir]
    cmd += ["-I" + p for p in REF_INCLUDES]
    cmd += ["-I" + os.path.join(ROOT, "include"), "-I" + rocm_include, "-I" + os.path.join(ROOT, "nixl_amd", "csrc", "plugin"),
            os.path.join(ROOT, "nixl_amd", "csrc", "plugin", "hip_backend.cpp")]
    _run(cmd)


def test_boundary_layout_equals_reference(shim_dir, tmp_path):
    probe = os.path.join(ROOT, "tests", "cpp", "abi_layout_probe.cpp")
    common = ["g++", "-std=c++20", "-Wno-invalid-offsetof"]
    _run(common + ["-I" + shim_dir] + ["-I" + p for p in REF_INCLUDES] + [probe, "-o", str(tmp_path / "probe_ref")])
    _run(common + ["-I" + os.path.join(ROOT, "include", "nixl"), probe, "-o", str(tmp_path / "probe_ours")])
    ref = _run([str(tmp_path / "probe_ref")])
    ours = _run([str(tmp_path / "probe_ours")])
    assert len(ref.splitlines()) >= 60
    assert ours == ref
