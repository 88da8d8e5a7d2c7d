"""In-tree build of libmxd_msda.so (hipcc, gfx950).  No GPU is needed to compile."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))


def build(force=True, jobs=8, verbose=False):
    """Compile the HIP sources under ``csrc/`` into ``lib/libmxd_msda.so``.  Returns its path."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), f"-j{jobs}"]
    if force:
        cmd.append("-B")
    res = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
        print(res.stderr)
    if res.returncode != 0:
        raise RuntimeError("building libmxd_msda.so failed")
    return os.path.join(_HERE, "lib", "libmxd_msda.so")
