"""Compile libpmx_hip.so (gfx950) with hipcc through csrc/Makefile."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpmx_hip.so")


def build(force=True, jobs=8):
    """Runs make; with force=True every object is rebuilt.  The `lint` target checks the assembly of
    the kernels with hand-scheduled loads for register hazards and fails the build when it finds one."""
    cmd = ["make", "-C", os.path.join(HERE, "csrc"), "-j%d" % jobs, "all", "lint"]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("build finished without producing %s" % LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build())
