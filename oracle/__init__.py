"""CPU oracle package (test infrastructure only: imported by tests/, the smoke check and bench.py's CPU baseline)."""
from .oracle import *  # noqa: F401,F403
