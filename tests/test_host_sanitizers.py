"""The library's C host code (generators, checker, plan builders, coalescer, thread registry) under AddressSanitizer and
UndefinedBehaviorSanitizer: tests/san/driver.c walks every entry point that needs no GPU over valid, boundary and
invalid arguments on a recorder thread, linked with the C files themselves and CPU stand-ins for the HIP layer."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "hcomm_amd", "csrc")
SAN = os.path.join(ROOT, "tests", "san")


@pytest.mark.skipif(shutil.which("gcc") is None, reason="no gcc")
def test_host_code_is_clean_under_asan_and_ubsan(tmp_path):
    exe = str(tmp_path / "san_driver")
    cmd = ["gcc", "-O1", "-g", "-std=c11", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-fno-omit-frame-pointer", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    cmd += [os.path.join(CSRC, f) for f in ("hg_api.c", "hg_batch.c", "hg_sched.c", "hg_plan.c", "hg_check.c")]
    cmd += [os.path.join(SAN, "stubs.c"), os.path.join(SAN, "driver.c"), "-o", exe, "-lpthread", "-lm"]
    build = subprocess.run(cmd, capture_output=True, text=True)
    if build.returncode != 0 and "sanitize" in build.stderr + build.stdout and "cannot find" in build.stderr:
        pytest.skip("the sanitizer runtimes are not installed")
    assert build.returncode == 0, build.stderr[-2000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe], capture_output=True, text=True, timeout=900, env=env)
    assert run.returncode == 0, (run.stdout[-1000:], run.stderr[-3000:])
    assert " bad 0" in run.stdout and "ERROR" not in run.stderr and "runtime error" not in run.stderr
    plans = int(run.stdout.split("plans")[1].split()[0])
    assert plans > 5000                                              # the walk did reach the plan builders


@pytest.mark.skipif(shutil.which("gcc") is None, reason="no gcc")
def test_host_code_is_clean_under_tsan_with_eight_host_threads(tmp_path):
    exe = str(tmp_path / "san_mt")
    cmd = ["gcc", "-O1", "-g", "-std=c11", "-fsanitize=thread", "-fno-omit-frame-pointer",
           "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    cmd += [os.path.join(CSRC, f) for f in ("hg_api.c", "hg_batch.c", "hg_sched.c", "hg_plan.c", "hg_check.c")]
    cmd += [os.path.join(SAN, "stubs.c"), os.path.join(SAN, "driver_mt.c"), "-o", exe, "-lpthread", "-lm"]
    build = subprocess.run(cmd, capture_output=True, text=True)
    if build.returncode != 0 and "cannot find" in build.stderr:
        pytest.skip("the sanitizer runtime is not installed")
    assert build.returncode == 0, build.stderr[-2000:]
    run = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    if "unexpected memory mapping" in run.stderr:                    # ThreadSanitizer cannot place its shadow here
        pytest.skip("ThreadSanitizer does not run in this environment")
    assert run.returncode == 0, (run.stdout[-1000:], run.stderr[-3000:])
    assert "threads 8 bad 0" in run.stdout and "ThreadSanitizer" not in run.stderr


@pytest.mark.skipif(shutil.which("gcc") is None, reason="no gcc")
def test_no_alloc_entry_point_allocates_nothing_on_the_host(tmp_path):
    """tests/san/driver_noalloc.c: every malloc / calloc / realloc / free the library's host code makes while
    HcommGfxAllReduceLocalReduceNoAlloc runs on an executing (not a recording) thread is counted through the linker's
    --wrap; the count must be zero over 120 calls that do reach their launches, and over refused calls."""
    exe = str(tmp_path / "noalloc_driver")
    cmd = ["gcc", "-O1", "-g", "-std=c11", "-DHG_STUB_GPU_PRESENT", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    cmd += [os.path.join(CSRC, f) for f in ("hg_api.c", "hg_batch.c", "hg_sched.c", "hg_plan.c", "hg_check.c")]
    cmd += [os.path.join(SAN, "stubs.c"), os.path.join(SAN, "driver_noalloc.c"), "-o", exe, "-lpthread", "-lm",
            "-Wl,--wrap=malloc", "-Wl,--wrap=calloc", "-Wl,--wrap=realloc", "-Wl,--wrap=free"]
    build = subprocess.run(cmd, capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-2000:]
    run = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, (run.stdout, run.stderr[-2000:])
    assert "calls 120 " in run.stdout and " allocations 0 frees 0 bad 0" in run.stdout, run.stdout
