"""Compile the HIP sources in ``research_amd/csrc`` into ``libpaged_attn.so``.

``python -m research_amd.build`` runs ``make`` with hipcc for gfx950; the
library lands next to the package's ``_lib.py``.  hipcc cross-compiles, so
this works on a machine without a GPU.
"""

from __future__ import annotations

import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")


def build(force: bool = False, jobs: int = 8) -> str:
    if force:
        subprocess.run(["make", "-C", CSRC, "clean"], check=True, stdout=subprocess.DEVNULL)
    proc = subprocess.run(["make", "-C", CSRC, f"-j{jobs}", "all"], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout)
        raise RuntimeError("building libpaged_attn.so failed")
    from . import _lib

    return _lib.LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
