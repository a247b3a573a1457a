"""Builds libyka.so with hipcc for gfx950 (cross-compiles without a GPU)."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))


def library_path() -> str:
    return os.path.join(_HERE, "libyka.so")


def build_library(force: bool = True, jobs: int = 4) -> str:
    """Runs make in csrc/.  force=True rebuilds from scratch (the build check compiles every time)."""
    csrc = os.path.join(_HERE, "csrc")
    if force:
        subprocess.run(["make", "-C", csrc, "clean"], check=True, stdout=subprocess.DEVNULL)
    proc = subprocess.run(["make", "-C", csrc, f"-j{jobs}"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building libyka.so failed:\n" + proc.stdout[-4000:])
    if not os.path.exists(library_path()):
        raise RuntimeError("make succeeded but libyka.so is missing")
    return library_path()


if __name__ == "__main__":
    print(build_library())
