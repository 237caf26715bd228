"""Alias of feather_amd.routines."""
from feather_amd.routines import *  # noqa: F401,F403
