"""Alias of feather_amd.packers.serial."""
from feather_amd.packers.serial import *  # noqa: F401,F403
