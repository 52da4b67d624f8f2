"""`pip install .` (the counterpart of the reference's setup.py, /root/reference/setup.py:4-21, a
torch CUDAExtension build): an offline install into a scratch directory, then the installed
packages are imported from there, in a fresh interpreter that cannot see this repository, with
both shared objects present and loadable (no GPU needed for that)."""
import os
import shutil
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_pip_install_into_a_target_directory_and_import_from_there(tmp_path):
    target = tmp_path / "site"
    leftovers = [p for p in ("build", "ds_splat_amd.egg-info") if not os.path.exists(os.path.join(ROOT, p))]
    try:
        r = subprocess.run([sys.executable, "-m", "pip", "install", "--no-build-isolation", "--no-deps", "--no-index",
                            "--quiet", "--target", str(target), "."], cwd=ROOT, capture_output=True, text=True,
                           timeout=900)
        assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    finally:
        for p in leftovers:                       # what the build left in the source tree
            shutil.rmtree(os.path.join(ROOT, p), ignore_errors=True)
    lib_dir = target / "ds_splat_amd" / "lib"
    names = sorted(os.listdir(lib_dir))
    assert "libdsx.so" in names and any(n.startswith("_dsx_torch") and n.endswith(".so") for n in names), names
    assert (target / "ds_splat" / "__init__.py").exists()
    code = (
        "import os, ds_splat, ds_splat_amd\n"
        "from ds_splat_amd import _native\n"
        "assert os.path.realpath(ds_splat.__file__).startswith(os.path.realpath(%r)), ds_splat.__file__\n"
        "assert os.path.realpath(_native.LIB_PATH).startswith(os.path.realpath(%r)), _native.LIB_PATH\n"
        "lib = _native.load(); ext = _native.load_torch_ext()\n"
        "assert lib.dsx_version() == ext.version() >= 100\n"
        "from ds_splat import GaussianRasterizationSettings, GaussianRasterizer\n"
        "print('installed ok')\n" % (str(target), str(target)))
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    env["PYTHONPATH"] = str(target)
    r = subprocess.run([sys.executable, "-c", code], cwd=str(tmp_path), env=env, capture_output=True, text=True,
                       timeout=600)
    assert r.returncode == 0 and "installed ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
