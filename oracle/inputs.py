"""The seeded synthetic inputs that the tests feed to the oracle and to the HIP path alike; the generators live in
nmtgminor_amd/synthetic.py, where the benchmark finds them without importing anything from this directory."""
from nmtgminor_amd.synthetic import *  # noqa: F401,F403
