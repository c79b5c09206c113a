"""Compiles the HIP sources in csrc/ into libomk_forest.so (gfx950), in-tree."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def build_library(force=True, jobs=4):
    """Runs make in csrc/.  With force the objects are rebuilt even when up to date."""
    cmd = ["make", "-C", os.path.join(HERE, "csrc"), "-j%d" % jobs]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    so = os.path.join(HERE, "libomk_forest.so")
    if not os.path.exists(so):
        raise RuntimeError("build finished without producing " + so)
    return so


if __name__ == "__main__":
    print(build_library())
