"""Compile ``libinfinirt.so``, ``libinfiniop.so`` and ``libinfinicore_ops.so`` for gfx950 with hipcc (no GPU needed)."""
from __future__ import annotations

import os
import subprocess
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
CSRC_DIR = PACKAGE_DIR / "csrc"
LIB_DIR = PACKAGE_DIR / "lib"
LIBRARIES = ("libinfinirt.so", "libinfiniop.so", "libinfinicore_ops.so")


def libraries_present() -> bool:
    return all((LIB_DIR / name).is_file() for name in LIBRARIES)


def build(force: bool = True, jobs: int | None = None, verbose: bool = False) -> None:
    """Run the Makefile in ``csrc/``. ``force`` rebuilds from scratch (``make clean`` first)."""
    jobs = jobs or min(8, os.cpu_count() or 1)
    if force:
        subprocess.run(["make", "-C", str(CSRC_DIR), "clean"], check=True, capture_output=not verbose)
    proc = subprocess.run(["make", "-C", str(CSRC_DIR), f"-j{jobs}"], capture_output=not verbose, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building the InfiniOP AMD libraries failed:\n" + (proc.stdout or "") + (proc.stderr or ""))
    if not libraries_present():
        raise RuntimeError(f"build finished but {LIBRARIES} are not in {LIB_DIR}")


if __name__ == "__main__":
    build(force=False, verbose=True)
