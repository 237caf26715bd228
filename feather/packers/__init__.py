"""Alias of feather_amd.packers."""
from feather_amd.packers import *  # noqa: F401,F403
