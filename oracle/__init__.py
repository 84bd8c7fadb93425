"""CPU checker for the OMMX decode-attention path (test infrastructure, never shipped)."""
from .ommx_oracle import *  # noqa: F401,F403
