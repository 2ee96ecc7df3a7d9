"""Name the reference's latency script imports (test.py:4): the double-channel backward."""
from .double_channel_bwd33 import *  # noqa: F401,F403
from .double_channel_bwd33 import bwd_33  # noqa: F401
