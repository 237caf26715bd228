"""Alias of feather_amd.routines.producers."""
from feather_amd.routines.producers import *  # noqa: F401,F403
