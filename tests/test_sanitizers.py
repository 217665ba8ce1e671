"""The CPU side under AddressSanitizer and UndefinedBehaviorSanitizer.

The oracle allocates per-thread score rows and indexes hand-rolled [B,H,S,Nq,d] layouts; `make -C oracle asan` builds it
with -fsanitize=address,undefined (undefined behaviour is fatal), and the whole of tests/test_oracle.py runs against that
build in a child process with libasan preloaded.  The bench + verify driver's host code (argument parsing, input fill,
file output: everything in front of its first HIP call) is built and run the same way, and so is the host side of the
library's C ABI (flash_api.hip: argument checks, split resolution, workspace sizing in long long / size_t), against which
tests/test_abi.py runs.  The reference's only counterpart is its CUDA_CHECK macro (src/main.cu:18-25).  No GPU needed;
sanitizers never see device code.
"""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _asan_env():
    libasan = subprocess.check_output(["gcc", "-print-file-name=libasan.so"], text=True).strip()
    if not os.path.isabs(libasan) or not os.path.exists(libasan):
        pytest.skip("gcc has no libasan.so here")
    env = dict(os.environ)
    # the sanitizer runtime has to come first among the preloaded libraries; whatever is preloaded already stays
    env["LD_PRELOAD"] = libasan + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
    # the interpreter itself is not built for leak checking; everything else stays fatal
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=0:exitcode=99"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    return env


def test_oracle_tests_pass_under_asan_and_ubsan():
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "asan"])
    lib = os.path.join(ROOT, "oracle", "liboracle_asan.so")
    env = _asan_env()
    env["FLASH_ORACLE_LIB"] = lib
    # the child really runs the instrumented build with the runtime loaded
    probe = ("import sys; sys.path.insert(0, %r)\n"
             "from oracle import cpu_oracle as co\n"
             "co.lib(); maps = open('/proc/self/maps').read()\n"
             "assert 'liboracle_asan.so' in maps and 'libasan' in maps, 'sanitizer build not loaded'\n"
             "import numpy as np\n"
             "co.normal_f16((1001,), 3, first=5); co.dropout_keep_mask(1, 2, 0.3, 1, 2, 33, 77)\n" % ROOT)
    r = subprocess.run([sys.executable, "-c", probe], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider",
                        os.path.join(ROOT, "tests", "test_oracle.py")], env=env, capture_output=True, text=True,
                       timeout=900, cwd=ROOT)
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-3000:])
    assert "passed" in r.stdout and "ERROR: AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr


def test_driver_host_code_under_asan_and_ubsan(tmp_path):
    drv = os.path.join(ROOT, "tests", "driver")
    subprocess.check_call(["make", "-s", "-C", drv, "flash_driver_asan"])
    exe = os.path.join(drv, "flash_driver_asan")
    env = _asan_env()
    env.pop("LD_PRELOAD")  # an executable built with -fsanitize links its runtime itself
    if os.environ.get("LD_PRELOAD"):
        env["LD_PRELOAD"] = os.environ["LD_PRELOAD"]

    def run(*args):
        return subprocess.run([exe, *args], env=env, capture_output=True, text=True, timeout=300)

    for args, rc in ((("--help",), 2), (("--no-such-flag",), 2), (("--seq", "0"), 2), (("--batch",), 2),
                     (("--fill", "gaussian"), 2)):
        r = run(*args)
        assert r.returncode == rc, (args, r.returncode, r.stderr[-2000:])
    # both fills and the file output, sizes that are no multiple of the generator's block of four
    for fill in ("reference", "normal"):
        f = tmp_path / f"{fill}.bin"
        r = run("--fill", fill, "--seed", "5", "--batch", "2", "--heads", "3", "--seq", "41", "--head-dim", "7",
                "--dump-inputs", str(f))
        assert r.returncode == 0, r.stderr[-3000:]
        assert os.path.getsize(f) == 3 * 2 * (2 * 3 * 41 * 7)


def test_library_host_side_under_asan_and_ubsan():
    """tests/test_abi.py (argument errors, split resolution for Nq = 1 and Nq > 1, workspace and stamp-buffer sizes, the
    heuristic table) against a build of the library whose host code is instrumented; the runtime is the compiler's own
    (hipcc is clang), preloaded in front of whatever is preloaded already."""
    csrc = os.path.join(ROOT, "flash_attn_amd", "csrc")
    subprocess.check_call(["make", "-s", "-C", csrc, "asan"])
    lib = os.path.join(ROOT, "flash_attn_amd", "lib", "libflash_attn_mi355_asan.so")
    clang = "/opt/rocm/lib/llvm/bin/clang"
    if not os.path.exists(clang):
        pytest.skip("no clang to ask for its sanitizer runtime")
    rt = subprocess.check_output([clang, "-print-file-name=libclang_rt.asan-x86_64.so"], text=True).strip()
    if not os.path.isabs(rt) or not os.path.exists(rt):
        pytest.skip("clang has no shared AddressSanitizer runtime here")
    env = dict(os.environ)
    env["LD_PRELOAD"] = rt + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
    env["ASAN_OPTIONS"] = "detect_leaks=0:exitcode=99"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    runner = ("import sys; sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
              "from flash_attn_amd import binding\n"
              "binding._LIB_PATH = %r\n"
              "binding.lib(); maps = open('/proc/self/maps').read()\n"
              "assert 'libflash_attn_mi355_asan.so' in maps and 'libclang_rt.asan' in maps, 'sanitizer build not loaded'\n"
              "import pytest\n"
              "sys.exit(pytest.main(['-x', '-q', '-p', 'no:cacheprovider', %r]))\n"
              % (ROOT, os.path.join(ROOT, "tests"), lib, os.path.join(ROOT, "tests", "test_abi.py")))
    r = subprocess.run([sys.executable, "-c", runner], env=env, capture_output=True, text=True, timeout=900, cwd=ROOT)
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-3000:])
    assert "passed" in r.stdout and "ERROR: AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr
