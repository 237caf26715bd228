"""Alias of feather_amd.routines.dot (reference module path)."""
from feather_amd.routines.dot import *  # noqa: F401,F403
