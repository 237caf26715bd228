"""Alias of feather_amd.packers.fp8 (reference module path)."""
from feather_amd.packers.fp8 import *  # noqa: F401,F403
