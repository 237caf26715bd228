"""Alias of feather_amd.packers.fp16 (reference module path)."""
from feather_amd.packers.fp16 import *  # noqa: F401,F403
