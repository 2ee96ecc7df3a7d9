"""Name the reference's latency script imports (test.py:3): the double-channel forward."""
from .double_channel_fwd32 import *  # noqa: F401,F403
from .double_channel_fwd32 import fwd_32  # noqa: F401
