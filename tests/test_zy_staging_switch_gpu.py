"""Kernels the library keeps behind environment switches that are read once per process (the register-staged flash
kernels of every head-dim class; the one-patch streaming forward kernel at head dim 128): their tests run again in a
child process that sets the switch.  Collected late on purpose: a slow start of a child must not hide other tests behind
a stop at the first failure."""
import pytest

pytestmark = pytest.mark.gpu


def test_register_staged_kernels_behind_the_environment_switch():
    """DLT_FLASH_SYNC_STAGING=1 (read once per process) keeps the register-staged kernels for every head-dim class:
    the flash test file and the flash sweeps of the fuzz file pass in a child process that sets it."""
    import os
    import subprocess
    import sys
    if os.environ.get("DLT_FLASH_SYNC_STAGING") == "1":
        pytest.skip("already running with the switch set")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, DLT_FLASH_SYNC_STAGING="1")
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", "tests/test_flash_gpu.py", "tests/test_fuzz_gpu.py", "-m", "gpu", "-x", "-q",
                        "-k", "flash", "-p", "no:cacheprovider"],
                       cwd=root, env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-1000:]
    assert " passed" in r.stdout and "failed" not in r.stdout, r.stdout[-500:]



def test_one_patch_streaming_forward_kernel_behind_the_environment_switch():
    """DLT_SWA2_SINGLE_PATCH=1 (read once per process) keeps the forward kernel with one patch per wave at head dim 128 on
    grids of more than 8 rows (without the switch it only runs on grids of up to 8 rows): the head-dim-128 token-grid
    tests pass in a child process that sets it."""
    import os
    import subprocess
    import sys
    if os.environ.get("DLT_SWA2_SINGLE_PATCH") == "1":
        pytest.skip("already running with the switch set")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, DLT_SWA2_SINGLE_PATCH="1")
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", "tests/test_swa_fwd_gpu.py", "tests/test_swa_tiles_gpu.py", "-m", "gpu", "-x", "-q",
                        "-k", "head_dim_128 or wider or small_tiles or head_dims", "-p", "no:cacheprovider"],
                       cwd=root, env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-1000:]
    assert " passed" in r.stdout and "failed" not in r.stdout, r.stdout[-500:]
