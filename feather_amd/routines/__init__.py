"""Routines on packed operands: GEMV, dot, flash / paged attention, ReLU, and the producers that
emit packed operands."""
from .gemv import *  # noqa: F401,F403
from .dot import *  # noqa: F401,F403
from .attention import *  # noqa: F401,F403
from .paged_attention import *  # noqa: F401,F403
from .activations import *  # noqa: F401,F403
from .producers import *  # noqa: F401,F403
