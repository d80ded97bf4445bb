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


def test_the_product_never_reaches_the_cpu_oracle():
    """The oracle is the checker of the tests: nothing that ships (the package, the headers,
    ``setup.py``) imports, links, loads or starts it, and the built libraries do not depend on it."""
    import re
    reach = re.compile(r"\b(?:import\s+oracle|from\s+oracle|fgs_oracle|libfgs_oracle)\b|[\"'/]oracle/")
    shipped = [os.path.join(ROOT, "setup.py")]
    for top in ("flashgs_amd", "include"):
        for folder, _, files in os.walk(os.path.join(ROOT, top)):
            shipped += [os.path.join(folder, f) for f in files
                        if f.endswith((".py", ".hip", ".cpp", ".h", ".hpp", ".inc"))]
    assert len(shipped) > 10
    for path in shipped:
        with open(path, errors="replace") as fh:
            hits = [line.strip() for line in fh if reach.search(line)]
        assert not hits, (path, hits)
    built = glob.glob(os.path.join(ROOT, "flashgs_amd", "lib", "*.so")) + glob.glob(os.path.join(ROOT, "flash_gaussian_splatting*.so"))
    assert built, "nothing built: run __graft_entry__.build() first"
    for lib in built:
        needed = subprocess.check_output(["readelf", "-d", lib], timeout=60).decode()
        assert "oracle" not in needed, lib
