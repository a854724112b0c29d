"""Public alias of the operator wrappers (same role as `vllm._custom_ops`)."""
from ._custom_ops import *  # noqa: F401,F403
from ._custom_ops import REGISTERED  # noqa: F401
