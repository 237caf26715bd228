"""Alias of feather_amd.routines.gemv (reference module path)."""
from feather_amd.routines.gemv import *  # noqa: F401,F403
