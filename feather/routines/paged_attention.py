"""Alias of feather_amd.routines.paged_attention (reference module path)."""
from feather_amd.routines.paged_attention import *  # noqa: F401,F403
