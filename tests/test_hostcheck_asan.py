"""AddressSanitizer run of the kernels' host build (global-memory bounds of every kernel)."""

import os
import subprocess
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))


def test_host_build_is_memory_clean():
    with tempfile.TemporaryDirectory() as tmp:
        exe = os.path.join(tmp, "driver")
        subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined",
                               "-fno-sanitize-recover=all", "-static-libasan", "-static-libubsan",
                               "-Wno-unknown-pragmas",
                               os.path.join(HERE, "hostcheck_asan_driver.cpp"), "-o", exe])
        # the sanitizer runtimes are linked statically, so the process environment
        # (including any preloaded library) is left exactly as it is
        proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                              timeout=600)
        assert proc.returncode == 0, proc.stdout[-4000:]
