"""Packers: fp16 -> packed FP8 / FP16 words (HIP kernels behind the reference's names)."""
from .fp8 import *  # noqa: F401,F403
from .fp16 import *  # noqa: F401,F403
from .serial import *  # noqa: F401,F403
