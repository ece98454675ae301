"""Every kernel the dispatcher can fall back to, on shapes the faster kernels
normally take: the debugging switches of the library (read once per process)
turn the faster paths off one at a time, and the same cases must still meet
the oracle.  One child process per switch, one after the other."""
from __future__ import annotations

import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SWITCHES = [
    None,                            # the default dispatch
    "SONAR_MARLIN_NO_FAST",          # the register-prefetch streaming kernel for every M <= 64
    "SONAR_MARLIN_NO_SLABS",         # no blocks of rows in the 16-row kernel
    "SONAR_MARLIN_NO_ROW_PAIRS",     # blocks of 16 rows only
    "SONAR_MARLIN_NO_HALF_WG",       # 8-wavefront workgroups only
    "SONAR_MARLIN_NO_NT_WEIGHTS",    # no non-temporal bit on the weight copies of large matrices
    "SONAR_MARLIN_SPLIT=1",          # no strip shared between workgroups
    "SONAR_MARLIN_NO_INLINE_SUM",    # shared strips summed by the fix-up launch
    "SONAR_MARLIN_NO_TILE",          # the streaming kernels in 64-row slabs for every M
    "SONAR_MARLIN_NO_WIDE_TILE",     # the eight-wavefront tile kernel where the wide one would run
    "SONAR_MARLIN_NO_128_ROW_TILES", # the wide tile kernel with 256-row tiles only
    "SONAR_MARLIN_NO_ASYNC_TILE",    # the register-staged tile kernel
    "SONAR_MARLIN_MAX_K_SPLITS=1",   # no split K in the tile kernel
    "SONAR_MARLIN_NO_TWO_TILE_SIZES",  # a short last round of tiles cut along K instead of a second launch of 128-row tiles
    "SONAR_MARLIN_NO_MOE_TILE",      # the grouped streaming kernel for 64-slot blocks
    "SONAR_MARLIN_NO_MOE_FAST",      # ... and for blocks of up to 32 slots
    "SONAR_MARLIN_NO_MOE_K_SPLIT",   # the grouped wide tile kernel never cuts its tiles along K
    "SONAR_MARLIN_NO_MOE_128_ROW_TILES",   # ... and computes the short ends of the experts' rows as 256-row tiles
    "SONAR_MARLIN_NO_MOE_PERMUTED_COPY",   # act-order experts: the gathering kernel although scratch has room
]


@pytest.mark.parametrize("switch", SWITCHES, ids=lambda s: s or "default")
def test_every_dispatch_path_meets_the_oracle(switch):
    env = dict(os.environ)
    if switch:
        name, _, value = switch.partition("=")
        env[name] = value or "1"
    out = subprocess.run([sys.executable, "-u", "-m", "tests.dispatch_paths_child"], cwd=ROOT, env=env,
                         capture_output=True, text=True, timeout=110)
    assert out.returncode == 0 and "all paths ok" in out.stdout, out.stdout[-1500:] + out.stderr[-1500:]
