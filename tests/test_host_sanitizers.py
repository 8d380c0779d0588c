"""Host code under AddressSanitizer / UBSan: the tile model, the enumeration and the weight packing of all three
algorithms are compiled with g++ (no GPU code is involved) and driven over a dozen shapes; every packed buffer is
allocated at exactly the size the library reports, so an overrun of the packing loops is caught."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_model_and_packing_are_clean_under_asan_and_ubsan(tmp_path):
    gxx = shutil.which("g++")
    if not gxx:
        pytest.skip("g++ not available")
    exe = str(tmp_path / "model_asan")
    # (the tile model compiles in the register report of the kernels, which the library's build leaves here)
    built = os.path.join(ROOT, "ppopp23-tdc_amd", "build")
    if not os.path.exists(os.path.join(built, "kernel_registers.inc")):
        pytest.skip("kernel_registers.inc is absent: build the library first (make -C ppopp23-tdc_amd/csrc)")
    build = subprocess.run(
        [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-static-libasan", "-static-libubsan",
         "-fno-omit-frame-pointer", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "ppopp23-tdc_amd", "csrc"), "-I" + built,
         os.path.join(ROOT, "tests", "host_sanitize_main.cpp"), os.path.join(ROOT, "ppopp23-tdc_amd", "csrc", "tile_model.cpp"),
         "-o", exe], capture_output=True, text=True, timeout=600)
    assert build.returncode == 0, build.stderr[-2000:]
    env = dict(os.environ)
    # (the sanitizer runtimes are linked statically, so the environment's library list does not matter to them)
    env["ASAN_OPTIONS"] = "detect_leaks=1:verify_asan_link_order=0"
    run = subprocess.run([exe], capture_output=True, text=True, timeout=900, env=env)
    assert run.returncode == 0, (run.stdout[-1500:], run.stderr[-3000:])
    assert "packed" in run.stdout and "ERROR" not in run.stderr
