"""Alias of feather_amd.routines.attention (reference module path)."""
from feather_amd.routines.attention import *  # noqa: F401,F403
