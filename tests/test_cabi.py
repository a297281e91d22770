"""CPU-side checks of the boundary: the shared library loads and exports every symbol that
include/turbofno.h declares; the codelet arithmetic (host build) matches a brute-force DFT."""
import ctypes
import os
import re
import subprocess

import turbofno_amd as tf

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "turbofno.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(turbofno_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 8
    L = ctypes.CDLL(tf.library_path())
    for n in names:
        assert hasattr(L, n), n


def test_abi_version_and_error_string_without_gpu():
    L = tf.lib()
    assert L.turbofno_abi_version() == 2
    assert L.turbofno_last_error_string() is not None
    # argument validation happens before any GPU call
    rc = L.turbofno_fused_fft_cgemm_ifft(8, 64, 64, 12, 1, 1, None, 1, 1.0, 0.0, 0.0, 0.0, None)
    assert rc == 1 and b"K=12" in L.turbofno_last_error_string()
    rc = L.turbofno_fused_fft_cgemm_ifft(11, 64, 64, 8, 1, 1, None, 1, 1.0, 0.0, 0.0, 0.0, None)
    assert rc == 2
    rc = L.turbofno_layer_2d(1, 256, 256, 8, 64, 1, 1, 1, 1.0, 0.0, None, 0, 0, None)
    assert rc == 3
    assert L.turbofno_layer_2d_workspace_bytes(16, 256, 256, 64, 64, 0) == 2 * 64 * 16 * 4096 * 8


def test_codelets_on_cpu(tmp_path):
    exe = str(tmp_path / "codelet_check")
    subprocess.run(["g++", "-O1", "-std=c++17", os.path.join(ROOT, "tests", "host", "codelet_check.cpp"), "-o", exe],
                   check=True)
    out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout
    assert out.strip().endswith("OK"), out


def test_group_transforms_with_their_exchange_layouts_on_cpu(tmp_path):
    """the device functions of group_fft.h, one host thread per lane and a barrier where the wavefront runs in lockstep:
    lengths 128 to 1024 forward and backward through the real LDS layouts, against a double-precision DFT"""
    exe = str(tmp_path / "group_lanes_check")
    subprocess.run(["g++", "-O1", "-std=c++17", "-pthread", os.path.join(ROOT, "tests", "host", "group_lanes_check.cpp"), "-o", exe],
                   check=True)
    out = subprocess.run([exe], check=True, capture_output=True, text=True, timeout=300).stdout
    assert out.strip().endswith("OK"), out


def test_cmake_package_builds_and_links(tmp_path):
    """the CMake side of the integration: the top-level CMakeLists.txt builds libturbofno.so for gfx950 (library target
    only), installs it with its package file, and a consumer that says find_package(turbofno) +
    target_link_libraries(... turbofno::turbofno) builds and runs (no GPU needed: it only asks for the ABI version and a
    size rule)"""
    import shutil
    import pytest
    if not shutil.which("cmake") or not os.path.exists("/opt/rocm/lib/llvm/bin/clang++"):
        pytest.skip("cmake or the ROCm clang is not installed")
    build, prefix, cons = str(tmp_path / "build"), str(tmp_path / "prefix"), tmp_path / "consumer"
    gen = ["-G", "Ninja"] if shutil.which("ninja") else []
    run = lambda *cmd: subprocess.run(list(cmd), check=True, capture_output=True, text=True, timeout=900)
    run("cmake", "-S", ROOT, "-B", build, *gen, "-DCMAKE_HIP_COMPILER=/opt/rocm/lib/llvm/bin/clang++", "-DTURBOFNO_BUILD_DRIVERS=OFF")
    run("cmake", "--build", build, "-j", "8")
    run("cmake", "--install", build, "--prefix", prefix)
    L = ctypes.CDLL(os.path.join(prefix, "lib", "libturbofno.so"))
    for n in declared_symbols():
        assert hasattr(L, n), n
    cons.mkdir()
    (cons / "CMakeLists.txt").write_text("cmake_minimum_required(VERSION 3.21)\nproject(consumer LANGUAGES CXX)\n"
                                         "find_package(turbofno REQUIRED)\nadd_executable(consumer main.cpp)\n"
                                         "target_link_libraries(consumer PRIVATE turbofno::turbofno)\n")
    (cons / "main.cpp").write_text('#include <turbofno.h>\n#include <cstdio>\nint main() { std::printf("%d %d\\n", '
                                   'turbofno_abi_version(), turbofno_query_2d_algo(16, 256, 256, 64, 64, 0)); return 0; }\n')
    run("cmake", "-S", str(cons), "-B", str(cons / "b"), "-Dturbofno_DIR=" + os.path.join(prefix, "lib", "cmake", "turbofno"))
    run("cmake", "--build", str(cons / "b"))
    out = run(str(cons / "b" / "consumer")).stdout.split()
    assert out == ["2", "2"], out
