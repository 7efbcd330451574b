"""Runs GPU test files on the CPU against the kernel sources (tests/hostsim): a rehearsal of indexing, masking,
launch arithmetic and the tests' own logic before a GPU is spent on them. Timing, memory ordering and performance
are outside what it can show.

    python tests/hostsim/rehearse.py tests/test_attention_gpu.py [-k expr] [any pytest option]

Environment: HOSTSIM_CUS (compute units the launch code sees, default 4; 256 mirrors the tile choices made on an
MI355X), HOSTSIM_DMA=late|early (timing model of the global -> LDS transfers), the library's own NMTG_* switches.
Cost: about 0.1 ms per 32x32x16 MFMA, so keep M N K below ~10^9 per case (select with -k).
"""
import os
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "tests"), HERE):
    if p not in sys.path:
        sys.path.insert(0, p)
import harness  # noqa: E402

if __name__ == "__main__":
    harness.install(setattr, fake_gpu=True)
    os.chdir(ROOT)
    sys.exit(pytest.main(["-q", "-p", "no:cacheprovider", "-m", "gpu", "--timeout", "300"] + sys.argv[1:]))
