"""Alias of feather_amd.routines.activations (reference module path)."""
from feather_amd.routines.activations import *  # noqa: F401,F403
