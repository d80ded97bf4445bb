"""``pip install .`` (FlashGS ``setup.py:32-48`` is the counterpart): the extension and the package
install into a directory outside the repository and load from there, the extension finding the
HIP library through its run path."""
import glob
import os
import shutil
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_pip_install_outside_the_repository(tmp_path):
    target = tmp_path / "site"
    env = dict(os.environ, FLASHGS_AMD_REUSE_BUILT="1")      # the binaries are built already (build step of the driver)
    before = set(glob.glob(os.path.join(ROOT, "build")) + glob.glob(os.path.join(ROOT, "*.egg-info")))
    try:
        subprocess.check_call([sys.executable, "-m", "pip", "install", "--quiet", "--no-build-isolation", "--no-deps",
                               "--no-index", "--target", str(target), ROOT], env=env, cwd=str(tmp_path), timeout=900)
    finally:      # pip builds in the source tree: leave it as it was
        for left in set(glob.glob(os.path.join(ROOT, "build")) + glob.glob(os.path.join(ROOT, "*.egg-info"))) - before:
            shutil.rmtree(left, ignore_errors=True)
    code = (
        "import os, torch\n"
        "import flash_gaussian_splatting as f\n"
        "import flashgs_amd\n"
        "from flashgs_amd import cabi\n"
        "print(os.path.dirname(os.path.abspath(f.__file__)))\n"
        "print(os.path.dirname(os.path.abspath(flashgs_amd.__file__)))\n"
        "print(cabi.LIB_PATH)\n"
        "print(cabi.load().fgs_abi_version(), f.ops.get_sort_buffer_size(1 << 20))\n"
        "libs = [l.split()[-1] for l in open('/proc/self/maps') if 'libflashgs_hip' in l]\n"
        "print(sorted(set(libs))[0])\n"
    )
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    env["PYTHONPATH"] = str(target)
    out = subprocess.check_output([sys.executable, "-c", code], env=env, cwd=str(tmp_path), timeout=600).decode().split("\n")
    assert out[0] == str(target)
    assert out[1] == str(target / "flashgs_amd")
    assert out[2] == str(target / "flashgs_amd" / "lib" / "libflashgs_hip.so")
    version, size = out[3].split()
    assert int(version) >= 1 and int(size) >= 12 << 20
    assert out[4] == str(target / "flashgs_amd" / "lib" / "libflashgs_hip.so")     # the one the extension mapped
