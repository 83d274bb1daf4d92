"""CPU oracle for the target-verify hot path (test infrastructure only).

Importable from tests, the smoke entry and the benchmark's cpu_baseline leg;
never from the shipped package.
"""
from . import dflash_oracle  # noqa: F401
from .c_binding import load_c_oracle  # noqa: F401
