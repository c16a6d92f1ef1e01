"""The configurations live in workloads.py at the repository root (bench.py uses them too)."""
from workloads import *  # noqa: F401,F403
from workloads import _seed  # noqa: F401
